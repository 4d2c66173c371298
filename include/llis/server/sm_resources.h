#pragma once
// Aggregate occupancy budget of the whole GPU, used by the block-level scheduler to decide whether the
// next kernel still "fits" beside what is already resident.
//
// Four pooled quantities, each = per-CU capacity x number of CUs: vector-register lanes, LDS bytes, wave
// slots (counted in threads) and resident workgroups.  acquire()/release() move `num` workgroups of the job's
// CURRENT stage in or out; job_fits() tests the job's NEXT stage against what is left.  The pooling and the
// call sequence follow reference include/llis/server/sm_resources.h:9-53 and src/server/sm_resources.cpp:6-111;
// what one workgroup is CHARGED is what a gfx950 compute unit actually sets aside for it (the reference
// charges regs x threads, threads and bytes as declared, which is the CUDA allocation model):
//   * a workgroup occupies whole wavefronts: ceil(threads / 64) waves of 64 lanes, whatever it declared;
//   * each wave gets its vector registers (architectural + accumulation registers, one unified file of 512 per
//     SIMD lane) in granules of 8;
//   * LDS is handed out in granules of 1280 bytes (320 dwords; 160 KiB per CU).
// The capacities come from llis_hip_get_device_caps() (256 CUs x {4 SIMDs x 512 registers x 64 lanes, 160 KiB LDS,
// 32 wave slots, 32 workgroups} on MI355X).  blocks_per_cu() is the closed form of the same model for one
// compute unit; it equals what the runtime's occupancy query returns for the kernel.

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

    // gfx950 allocation units.
    static constexpr long long kWaveLanes = 64;         // lanes of a wavefront
    static constexpr long long kVgprGranule = 8;        // registers per allocation step, per lane
    static constexpr long long kLdsGranule = 1280;      // bytes per allocation step
    static constexpr long long kSimdsPerCu = 4;
    static constexpr long long kVgprsPerSimdLane = 512; // unified register file, per lane
    static constexpr long long kMaxWavesPerSimd = 8;
    static constexpr long long kMaxBlocksPerCu = 32;    // one-wave workgroups can take every wave slot

    static long long round_up(long long v, long long g) { return (v + g - 1) / g * g; }
    // What one workgroup takes out of each pool.
    static long long wg_threads(long long threads) { return round_up(threads, kWaveLanes); }
    static long long wg_regs(long long threads, long long regs_per_thread) { return wg_threads(threads) * round_up(regs_per_thread, kVgprGranule); }
    static long long wg_lds(long long lds_bytes) { return round_up(lds_bytes, kLdsGranule); }

    // Workgroups of this shape that one gfx950 compute unit holds at once: waves per SIMD by registers (at most 8),
    // times 4 SIMDs, divided by the workgroup's waves; then LDS; then the workgroup slots.
    static unsigned blocks_per_cu(unsigned threads, unsigned regs_per_thread, unsigned lds_bytes, unsigned lds_per_cu = 160 * 1024,
                                  unsigned max_blocks_per_cu = 32);

    bool job_fits(job::Job* job) const {
        const long long blocks = job->get_num_blocks();
        const long long threads = job->get_num_threads_per_block();
        return nregs_ >= wg_regs(threads, job->get_num_registers_per_thread()) * blocks &&
               smem_ >= wg_lds(job->get_smem_size_per_block()) * blocks && nthrs_ >= wg_threads(threads) * blocks && nblocks_ >= blocks;
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

// SmResources::blocks_per_cu for callers in other languages.
extern "C" unsigned llis_sm_resources_blocks_per_cu(unsigned threads, unsigned regs_per_thread, unsigned lds_bytes, unsigned lds_per_cu,
                                                    unsigned max_blocks_per_cu);
