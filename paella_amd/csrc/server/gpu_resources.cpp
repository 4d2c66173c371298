#include <llis/server/gpu_resources.h>
#include <llis/server/profiler.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <stdexcept>

namespace llis {
namespace server {

GpuResources::GpuResources() {
    llis_hip_device_caps caps;
    LLIS_CHECK_HIP(llis_hip_get_device_caps(&caps));
    init((unsigned)caps.num_cus, caps.num_cus % 8 == 0 ? 8u : 1u, caps.vgprs_per_cu, caps.lds_bytes_per_cu, caps.max_threads_per_cu, caps.max_blocks_per_cu);
}

GpuResources::GpuResources(unsigned num_cus, unsigned num_xcds, long long regs_per_cu, long long smem_per_cu, long long threads_per_cu,
                           long long blocks_per_cu) {
    init(num_cus, num_xcds, regs_per_cu, smem_per_cu, threads_per_cu, blocks_per_cu);
}

void GpuResources::init(unsigned num_cus, unsigned num_xcds, long long regs, long long smem, long long threads, long long blocks) {
    if (num_cus == 0 || num_xcds == 0 || num_cus % num_xcds != 0) throw std::invalid_argument("GpuResources: compute units must divide evenly into XCDs");
    if (num_cus > job::Job::kMaxCuIds) throw std::invalid_argument("GpuResources: more compute units than a message's id byte can name");
    cus_.assign(num_cus, SmResources(regs, smem, threads, blocks));
    total_ = SmResources(regs * num_cus, smem * num_cus, threads * num_cus, blocks * num_cus);
    num_xcds_ = num_xcds;
    cus_per_xcd_ = num_cus / num_xcds;
    next_cu_.assign(num_xcds, 0);
}

void GpuResources::acquire(unsigned cu, job::Job* job, int num) {
    SmResources& r = cus_.at(cu);
    const bool before = r.is_full();
    r.acquire(job, num);
    if (!before && r.is_full()) ++num_full_cus_;
    total_.acquire(job, num);
}

void GpuResources::release(unsigned cu, job::Job* job, int num) {
    SmResources& r = cus_.at(cu);
    const bool before = r.is_full();
    r.release(job, num);
    if (before && !r.is_full()) --num_full_cus_;
    total_.release(job, num);
}

bool GpuResources::job_fits(job::Job* job) const {
    const unsigned blocks = job->get_num_blocks();
    for (unsigned x = 0; x < num_xcds_; ++x) {
        // workgroups x, x + xcds, x + 2 xcds, ... (counted from the XCD the next dispatch starts on)
        const unsigned lane = (x + num_xcds_ - next_xcd_) % num_xcds_;
        const unsigned share = blocks > lane ? (blocks - lane + num_xcds_ - 1) / num_xcds_ : 0;
        unsigned room = 0;
        for (unsigned c = x * cus_per_xcd_; c < (x + 1) * cus_per_xcd_ && room < share; ++c) room += cus_[c].num_blocks(job);
        if (room < share) return false;
    }
    return true;
}

void GpuResources::choose_cus(job::Job* job) {
    const unsigned blocks = job->get_cur_num_blocks();
    for (unsigned i = 0; i < blocks; ++i) {
        const unsigned x = (next_xcd_ + i) % num_xcds_;
        // the compute unit of that XCD with the most free workgroup slots; ties go round
        unsigned best = 0;
        long long best_room = -(1ll << 62);
        for (unsigned k = 0; k < cus_per_xcd_; ++k) {
            const unsigned c = x * cus_per_xcd_ + (next_cu_[x] + k) % cus_per_xcd_;
            const long long room = cus_[c].is_full() ? -1 : cus_[c].free_threads();
            if (room > best_room) {
                best_room = room;
                best = c;
            }
        }
        next_cu_[x] = (best % cus_per_xcd_ + 1) % cus_per_xcd_;
        acquire(best, job, 1);   // may over-subscribe the compute unit: the hardware would queue that workgroup
        job->add_predicted_smid(best);
    }
    next_xcd_ = (next_xcd_ + blocks) % num_xcds_;
}

void GpuResources::observe_block_start(job::Job* job, unsigned cu) {
    if (cu >= cus_.size()) return;
    if (job->has_predicted_smid(cu)) job->dec_predicted_smid(cu);
    else acquire(cu, job, 1);
}

void GpuResources::release_predicted(job::Job* job, unsigned num) {
    const unsigned* predicted = job->get_predicted_smid_nums();
    for (unsigned c = 0; c < cus_.size() && num > 0; ++c) {
        const unsigned n = predicted[c] < num ? predicted[c] : num;
        if (n == 0) continue;
        release(c, job, (int)n);
        for (unsigned i = 0; i < n; ++i) job->dec_predicted_smid(c);
        num -= n;
    }
}

unsigned GpuResources::reconcile(job::Job* job, unsigned* wrong_cus) {
    const unsigned* predicted = job->get_predicted_smid_nums();
    unsigned wrong = 0, cus = 0;
    for (unsigned c = 0; c < cus_.size(); ++c) {
        const unsigned n = predicted[c];
        if (n == 0) continue;
        wrong += n;
        ++cus;
        release(c, job, (int)n);
    }
    job->clear_predicted_smids();
    if (wrong_cus) *wrong_cus = cus;
    if (profiler_) profiler_->record_kernel_block_mis_alloc(job->get_cur_num_blocks(), wrong, cus);
    return wrong;
}

}  // namespace server
}  // namespace llis
