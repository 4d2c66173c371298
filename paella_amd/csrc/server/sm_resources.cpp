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
    // Register lanes and wave slots of a compute unit in the hardware's own units (the runtime's device properties
    // carry a CUDA-shaped "registers per multiprocessor" of 65536, half of what the four SIMDs hold, and 2 for the
    // resident workgroups per compute unit, where one-wave workgroups can fill all 32 wave slots).
    init(cus * kSimdsPerCu * kVgprsPerSimdLane * kWaveLanes, cus * caps.lds_bytes_per_cu, cus * kSimdsPerCu * kMaxWavesPerSimd * kWaveLanes,
         cus * kMaxBlocksPerCu);
}

void SmResources::init(long long nregs, long long smem, long long nthrs, long long nblocks) {
    nregs_ = max_nregs_ = nregs;
    smem_ = max_smem_ = smem;
    nthrs_ = max_nthrs_ = nthrs;
    nblocks_ = max_nblocks_ = nblocks;
    max_resources_dot_prod_ = (double)nregs * (double)nregs + (double)nthrs * (double)nthrs + (double)smem * (double)smem;
}

unsigned SmResources::blocks_per_cu(unsigned threads, unsigned regs_per_thread, unsigned lds_bytes, unsigned lds_per_cu, unsigned max_blocks_per_cu) {
    if (threads == 0) return 0;
    const long long waves_per_wg = wg_threads(threads) / kWaveLanes;
    long long waves_per_simd = kMaxWavesPerSimd;
    if (regs_per_thread > 0) waves_per_simd = std::min(waves_per_simd, kVgprsPerSimdLane / round_up(regs_per_thread, kVgprGranule));
    long long n = kSimdsPerCu * waves_per_simd / waves_per_wg;
    if (lds_bytes > 0) n = std::min(n, (long long)lds_per_cu / wg_lds(lds_bytes));
    n = std::min(n, (long long)max_blocks_per_cu);
    return n > 0 ? (unsigned)n : 0u;
}

void SmResources::acquire(job::Job* job, int num) {
    const long long threads = job->get_cur_num_threads_per_block();
    nregs_ -= wg_regs(threads, job->get_cur_num_registers_per_thread()) * num;
    nthrs_ -= wg_threads(threads) * num;
    smem_ -= wg_lds(job->get_cur_smem_size_per_block()) * num;
    nblocks_ -= num;
    if (profiler_) profiler_->record_resource_event(job, (unsigned)num, Profiler::ResourceEvent::ACQUIRE);
}

void SmResources::release(job::Job* job, int num) {
    const long long threads = job->get_cur_num_threads_per_block();
    nregs_ += wg_regs(threads, job->get_cur_num_registers_per_thread()) * num;
    nthrs_ += wg_threads(threads) * num;
    smem_ += wg_lds(job->get_cur_smem_size_per_block()) * num;
    nblocks_ += num;
    if (profiler_) profiler_->record_resource_event(job, (unsigned)num, Profiler::ResourceEvent::RELEASE);
}

double SmResources::dot(job::Job* job) const {
    const long long threads = job->get_cur_num_threads_per_block();
    return (double)nregs_ * (double)wg_regs(threads, job->get_cur_num_registers_per_thread()) + (double)nthrs_ * (double)wg_threads(threads) +
           (double)smem_ * (double)wg_lds(job->get_smem_size_per_block());
}

double SmResources::dot_normalized(job::Job* job) const { return dot(job) / max_resources_dot_prod_; }

unsigned SmResources::num_blocks(job::Job* job) const {
    if (is_full()) return 0;
    long long n = nblocks_;
    const long long threads = job->get_num_threads_per_block();
    if (threads > 0) {
        const long long regs_per_block = wg_regs(threads, job->get_num_registers_per_thread());
        if (regs_per_block > 0) n = std::min(n, nregs_ / regs_per_block);
        n = std::min(n, nthrs_ / wg_threads(threads));
    }
    if (job->get_smem_size_per_block() > 0) n = std::min(n, smem_ / wg_lds(job->get_smem_size_per_block()));
    return n > 0 ? (unsigned)n : 0u;
}

float SmResources::normalize_resources(job::Job* job) const {
    const long long threads = job->get_num_threads_per_block();
    const float blocks = (float)job->get_num_blocks();
    const float per_block = (float)wg_regs(threads, job->get_num_registers_per_thread()) / (float)max_nregs_ + (float)wg_threads(threads) / (float)max_nthrs_ +
                            (float)wg_lds(job->get_smem_size_per_block()) / (float)max_smem_;
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

// C entry point of the per-compute-unit closed form, for checks written in other languages.
extern "C" unsigned llis_sm_resources_blocks_per_cu(unsigned threads, unsigned regs_per_thread, unsigned lds_bytes, unsigned lds_per_cu,
                                                    unsigned max_blocks_per_cu) {
    return llis::server::SmResources::blocks_per_cu(threads, regs_per_thread, lds_bytes, lds_per_cu, max_blocks_per_cu);
}
