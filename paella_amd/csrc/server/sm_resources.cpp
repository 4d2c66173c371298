#include <llis/server/profiler.h>
#include <llis/server/sm_resources.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <algorithm>

namespace llis {
namespace server {

SmResources::SmResources(long long nregs, long long smem, long long nthrs, long long nblocks) { init(nregs, smem, nthrs, nblocks); }

SmResources::SmResources() {
    llis_hip_device_caps caps;
    LLIS_CHECK_HIP(llis_hip_get_device_caps(&caps));
    const long long cus = caps.num_cus;
    init(cus * caps.vgprs_per_cu, cus * caps.lds_bytes_per_cu, cus * caps.max_threads_per_cu, cus * caps.max_blocks_per_cu);
}

void SmResources::init(long long nregs, long long smem, long long nthrs, long long nblocks) {
    nregs_ = max_nregs_ = nregs;
    smem_ = max_smem_ = smem;
    nthrs_ = max_nthrs_ = nthrs;
    nblocks_ = max_nblocks_ = nblocks;
    max_resources_dot_prod_ = (double)nregs * (double)nregs + (double)nthrs * (double)nthrs + (double)smem * (double)smem;
}

void SmResources::acquire(job::Job* job, int num) {
    const long long threads = job->get_cur_num_threads_per_block();
    nregs_ -= (long long)job->get_cur_num_registers_per_thread() * threads * num;
    nthrs_ -= threads * num;
    smem_ -= (long long)job->get_cur_smem_size_per_block() * num;
    nblocks_ -= num;
    if (profiler_) profiler_->record_resource_event(job, (unsigned)num, Profiler::ResourceEvent::ACQUIRE);
}

void SmResources::release(job::Job* job, int num) {
    const long long threads = job->get_cur_num_threads_per_block();
    nregs_ += (long long)job->get_cur_num_registers_per_thread() * threads * num;
    nthrs_ += threads * num;
    smem_ += (long long)job->get_cur_smem_size_per_block() * num;
    nblocks_ += num;
    if (profiler_) profiler_->record_resource_event(job, (unsigned)num, Profiler::ResourceEvent::RELEASE);
}

double SmResources::dot(job::Job* job) const {
    const double threads = job->get_cur_num_threads_per_block();
    return (double)nregs_ * (double)job->get_cur_num_registers_per_thread() * threads + (double)nthrs_ * threads +
           (double)smem_ * (double)job->get_smem_size_per_block();
}

double SmResources::dot_normalized(job::Job* job) const { return dot(job) / max_resources_dot_prod_; }

unsigned SmResources::num_blocks(job::Job* job) const {
    if (is_full()) return 0;
    long long n = nblocks_;
    const long long threads = job->get_num_threads_per_block();
    if (threads > 0) {
        const long long regs_per_block = (long long)job->get_num_registers_per_thread() * threads;
        if (regs_per_block > 0) n = std::min(n, nregs_ / regs_per_block);
        n = std::min(n, nthrs_ / threads);
    }
    if (job->get_smem_size_per_block() > 0) n = std::min(n, smem_ / (long long)job->get_smem_size_per_block());
    return n > 0 ? (unsigned)n : 0u;
}

float SmResources::normalize_resources(job::Job* job) const {
    const float threads = (float)job->get_num_threads_per_block();
    const float blocks = (float)job->get_num_blocks();
    const float per_block = (float)job->get_num_registers_per_thread() * threads / (float)max_nregs_ + threads / (float)max_nthrs_ +
                            (float)job->get_smem_size_per_block() / (float)max_smem_;
    return per_block * blocks + blocks / (float)max_nblocks_;
}

double SmResources::occupancy() const {
    const double t = 1. - (double)nthrs_ / (double)max_nthrs_;
    const double s = 1. - (double)smem_ / (double)max_smem_;
    const double r = 1. - (double)nregs_ / (double)max_nregs_;
    return std::max(t, std::max(s, r));
}

}  // namespace server
}  // namespace llis
