#pragma once
// Aggregate occupancy budget of the whole GPU, used by the block-level scheduler to decide whether the
// next kernel still "fits" beside what is already resident.
//
// Four pooled quantities, each = per-CU capacity x number of CUs: vector registers (counted per thread,
// i.e. registers/thread x threads/workgroup x workgroups), LDS bytes, resident threads, resident
// workgroups.  acquire()/release() move `num` workgroups of the job's CURRENT stage in or out;
// job_fits() tests the job's NEXT stage against what is left.  The arithmetic follows reference
// include/llis/server/sm_resources.h:9-53 and src/server/sm_resources.cpp:6-111; the capacities come from
// llis_hip_get_device_caps() (256 CUs, 160 KiB LDS per CU on MI355X) instead of cudaDeviceProp.

#include <llis/job/job.h>

namespace llis {
namespace server {

class Profiler;

class SmResources {
  public:
    // Totals for the whole device.
    SmResources(long long nregs, long long smem, long long nthrs, long long nblocks);
    // Queries the current device.
    SmResources();

    void acquire(job::Job* job, int num);
    void release(job::Job* job, int num);

    bool job_fits(job::Job* job) const {
        const long long blocks = job->get_num_blocks();
        const long long threads = job->get_num_threads_per_block();
        return nregs_ >= (long long)job->get_num_registers_per_thread() * threads * blocks &&
               smem_ >= (long long)job->get_smem_size_per_block() * blocks && nthrs_ >= threads * blocks && nblocks_ >= blocks;
    }

    bool is_full() const { return nregs_ <= 0 || smem_ <= 0 || nthrs_ <= 0 || nblocks_ <= 0; }

    // How many workgroups of the job's next stage fit right now.
    unsigned num_blocks(job::Job* job) const;
    // Inner product of the free vector with the job's per-workgroup demand (packing heuristics).
    double dot(job::Job* job) const;
    double dot_normalized(job::Job* job) const;
    // Demand of the job's next stage as a fraction of the whole device, summed over the four resources.
    float normalize_resources(job::Job* job) const;
    // Largest used fraction among threads, LDS and registers.
    double occupancy() const;

    long long free_regs() const { return nregs_; }
    long long free_smem() const { return smem_; }
    long long free_threads() const { return nthrs_; }
    long long free_blocks() const { return nblocks_; }

    void set_profiler(Profiler* profiler) { profiler_ = profiler; }

  private:
    void init(long long nregs, long long smem, long long nthrs, long long nblocks);

    long long nregs_ = 0, smem_ = 0, nthrs_ = 0, nblocks_ = 0;
    long long max_nregs_ = 0, max_smem_ = 0, max_nthrs_ = 0, max_nblocks_ = 0;
    double max_resources_dot_prod_ = 0;
    Profiler* profiler_ = nullptr;
};

}  // namespace server
}  // namespace llis
