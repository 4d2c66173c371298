#pragma once
// Per-compute-unit occupancy model with an XCD-aware placement prediction.
//
// The reference sketches this for NVIDIA parts as GpuResources (reference include/llis/server/gpu_resources.h:10-58,
// src/server/gpu_resources.cpp:9-96: one SmResources per SM, a fixed SM-to-GPC table, choose_sms() spreading a kernel's
// blocks over GPCs) and never builds it into a scheduler it ships.  Here it is built for MI355X: 256 compute units in 8
// XCDs of 32, and the dispatch rule the hardware follows -- workgroup i of a dispatch goes to XCD (i mod 8), inside the
// XCD to the compute unit with the most room -- so a kernel "fits" only if every XCD can take its share, which the pooled
// budget of SmResources cannot express.
//
// The compute unit a workgroup really ran on comes back in InstrumentInfo.smid from the un-aggregated hooks
// (llis/job/instrument.h: XCD in the top three bits); observe_block_start() reconciles it with the prediction the way
// reference src/server/scheduler_full.cpp:98-121 does, and hands the miss counts to the profiler's
// kernel_block_mis_alloc record.

#include <llis/job/job.h>
#include <llis/server/sm_resources.h>

#include <vector>

namespace llis {
namespace server {

class Profiler;

class GpuResources {
  public:
    // Queries the current device (8 XCDs assumed when the compute-unit count is a multiple of 8, else 1).
    GpuResources();
    // Explicit topology and per-compute-unit capacities (tests, other parts).
    GpuResources(unsigned num_cus, unsigned num_xcds, long long regs_per_cu, long long smem_per_cu, long long threads_per_cu, long long blocks_per_cu);

    void acquire(unsigned cu, job::Job* job, int num);
    void release(unsigned cu, job::Job* job, int num);

    // Every XCD can take its share of the job's next stage (share of XCD x = number of i < blocks with i mod xcds == x).
    bool job_fits(job::Job* job) const;

    unsigned get_num_cus() const { return (unsigned)cus_.size(); }
    unsigned get_num_xcds() const { return num_xcds_; }
    unsigned xcd_of(unsigned cu) const { return cu / cus_per_xcd_; }
    bool is_full() const { return num_full_cus_ >= cus_.size(); }
    unsigned num_full_cus() const { return num_full_cus_; }
    const SmResources& cu(unsigned i) const { return cus_[i]; }
    const SmResources& total() const { return total_; }

    // Predicts where the workgroups of the stage the job is about to run will land, acquires those compute units and
    // records the prediction in the job (Job::add_predicted_smid).  Call after the job's current stage is set.
    void choose_cus(job::Job* job);

    // A workgroup of the job's running stage reported compute unit `cu`.  Predicted there: the prediction is consumed;
    // otherwise the compute unit is acquired now.  An id beyond the topology is left out of the books (start and finish alike).
    void observe_block_start(job::Job* job, unsigned cu);
    // All workgroups of the stage have started: predictions that never came true are given back.  Returns the number
    // of mispredicted workgroups and stores the number of compute units they were predicted on; both go to the profiler.
    unsigned reconcile(job::Job* job, unsigned* wrong_cus);
    // A workgroup of the job's running stage finished on compute unit `cu`.
    void observe_block_finish(job::Job* job, unsigned cu) {
        if (cu < cus_.size()) release(cu, job, 1);
    }
    // `num` workgroups of the job's running stage finished and nothing says where (aggregated hooks): the prediction is all
    // there is, so they are released where they were predicted, lowest compute unit first.
    void release_predicted(job::Job* job, unsigned num);

    double dot(job::Job* job) const { return total_.dot(job); }
    double dot_normalized(job::Job* job) const { return total_.dot_normalized(job); }
    float normalize_resources(job::Job* job) const { return total_.normalize_resources(job); }

    void set_profiler(Profiler* profiler) { profiler_ = profiler; }

  private:
    void init(unsigned num_cus, unsigned num_xcds, long long regs, long long smem, long long threads, long long blocks);

    std::vector<SmResources> cus_;
    SmResources total_{0, 0, 0, 0};
    unsigned num_xcds_ = 1, cus_per_xcd_ = 1;
    unsigned num_full_cus_ = 0;
    std::vector<unsigned> next_cu_;   // per XCD: where the search for the roomiest compute unit starts (ties rotate)
    unsigned next_xcd_ = 0;           // XCD of the next dispatch's first workgroup
    Profiler* profiler_ = nullptr;
};

}  // namespace server
}  // namespace llis
