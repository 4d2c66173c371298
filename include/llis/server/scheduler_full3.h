#pragma once
// "full3": the Paella policy.
//
//  * Kernel-by-kernel dispatch: a job re-enters the queue after each of its stages completes.
//  * Priority = minus the job's remaining work (sum over not-yet-queued stages of learned length x
//    resource), i.e. shortest remaining processing time first.
//  * Fairness between job types with deficit counters: every dispatch charges the dispatched type 1 and
//    credits every active type 1/num_types; when the most-starved type's deficit reaches the threshold
//    its best job is served instead of the globally best one.
//  * Admission: a kernel is issued if its whole grid fits into what the occupancy model says is free;
//    otherwise it may still be issued as an "unfit" kernel while fewer than `extra_kernels` such kernels
//    are waiting to become fully resident (bounded over-subscription keeps the GPU's own queue short).
//
//  * With --placement per_cu the occupancy model is the per-compute-unit one (llis/server/gpu_resources.h): a kernel fits
//    if every XCD has room for its share of the grid, its workgroups are charged to the compute units the model predicts,
//    and for kernels that report through the un-aggregated hooks the prediction is reconciled with the compute unit every
//    start message names (reference src/server/scheduler_full.cpp:98-121 did that for an older scheduler; the reference's
//    full3 never got it).  Kernels with aggregated hooks are released where they were predicted.
//
// Policy and bookkeeping follow reference include/llis/server/scheduler_full3.h:26-269 and
// src/server/scheduler_full3.cpp:25-478.

#include <llis/server/gpu_resources.h>
#include <llis/server/scheduler.h>
#include <llis/server/sm_resources.h>

#include <cstdint>
#include <memory>
#include <set>
#include <vector>

namespace llis {
namespace server {

// Priority queue of jobs with per-type fairness.  Ties are served first-in first-out.
class JobQueue {
  public:
    explicit JobQueue(double unfairness_threshold) : unfairness_threshold_(unfairness_threshold) {}

    void push(job::Job* job);
    job::Job* top();   // queue must not be empty
    job::Job* pop();   // queue must not be empty
    bool empty() const { return all_.empty(); }
    size_t size() const { return all_.size(); }

    double threshold() const { return unfairness_threshold_; }

  private:
    struct JobKey {
        double priority;
        uint64_t seq;   // insertion order, breaks ties
        job::Job* job;
        bool operator<(const JobKey& o) const { return priority != o.priority ? priority > o.priority : seq < o.seq; }
    };
    struct TypeKey {
        double deficit;
        uint64_t seq;
        unsigned type_id;
        bool operator<(const TypeKey& o) const { return deficit != o.deficit ? deficit > o.deficit : seq < o.seq; }
    };
    struct TypeState {
        bool known = false;       // false: never seen, or reset because its last queued job left
        double deficit = 0;       // meaningful while the type is in active_types_
        uint64_t seq = 0;
        std::set<JobKey> jobs;
    };

    // The job the policy would serve now, and the type it belongs to.
    const JobKey& select(unsigned* type_id) const;

    double unfairness_threshold_;
    double new_type_deficit_ = 0;   // deficit a type starts with when it (re)appears
    unsigned num_types_ = 0;        // types that currently have queued jobs
    uint64_t next_seq_ = 0;

    std::set<JobKey> all_;
    std::vector<TypeState> types_;
    std::set<TypeKey> active_types_;  // most starved (largest deficit) first
};

class SchedulerFull3 : public StreamPoolScheduler {
  public:
    explicit SchedulerFull3(const SchedulerOptions& options);
    // For tests: an explicit occupancy budget instead of the device's.
    SchedulerFull3(const SchedulerOptions& options, const SmResources& budget);
    // For tests: per-compute-unit placement (options.per_cu_placement) over an explicit topology instead of the device's.
    SchedulerFull3(const SchedulerOptions& options, std::unique_ptr<GpuResources> per_cu);

    void set_server(Server* server) override;
    void handle_new_job(std::unique_ptr<job::Job> job) override;

  protected:
    void handle_block_start(job::Job* job, unsigned num) override;
    void handle_block_finish(job::Job* job, unsigned num) override;
    void handle_mem_finish(job::Job* job) override;

  private:
    void schedule_job();
    void requeue_or_finish(job::Job* job);
    double take_priority(job::Job* job) const;

    JobQueue job_queue_;
    SmResources gpu_resources_;
    std::unique_ptr<GpuResources> per_cu_;   // options.per_cu_placement: admission and accounting per compute unit instead
    int num_outstanding_kernels_ = 0;
};

}  // namespace server
}  // namespace llis
