#pragma once
// Server-side recorder behind the PROFILER_CMD messages.  The wire protocol (sub-command enum, SAVE
// carrying a path prefix) follows reference src/server/profiler.cpp:10-67 so a client's ProfilerClient
// keeps working; recording covers kernel info, per-job event timelines, run_next() times and resource events,
// written on SAVE as <prefix>_kernel_info.txt, _job_events.txt, _run_next_times.txt and _resource_events.txt in
// the reference's line formats (reference src/server/profiler.cpp:76-131), plus _block_exec_times.txt when the
// server runs with --measure_block_time (entry and exit clock of every workgroup, 24 bits each, 10 ns units).
// _kernel_block_mis_alloc.txt holds what GpuResources::reconcile() reports (the reference only writes it from a
// scheduler it does not build); it is empty when no per-compute-unit model is in use.

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/job/job.h>

#include <chrono>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace llis {
namespace server {

class Profiler {
  public:
    using TimePoint = std::chrono::steady_clock::time_point;

    enum class JobEvent { JOB_SUBMITTED, KERNEL_SCHED_START, KERNEL_SCHED_ABORT, KERNEL_SUBMIT_START, KERNEL_SUBMIT_END, KERNEL_FINISHED, JOB_FINISHED };
    enum class ResourceEvent { ACQUIRE, RELEASE, QUEUED };

    explicit Profiler(ipc::ShmChannelCpuReader* c2s_channel) : c2s_channel_(c2s_channel) {}

    // Consumes one PROFILER_CMD body from the request ring.
    void handle_cmd();
    void save(const std::string& path_prefix);

    bool recording_kernel_info() const { return kernel_info_flag_; }
    bool recording_job_events() const { return job_events_flag_; }

    void record_kernel_info(TimePoint start, TimePoint end, unsigned num_blocks, unsigned num_threads_per_block, unsigned smem_size_per_block,
                            unsigned num_registers_per_thread, double priority, unsigned job_ref_id);
    void record_job_event(JobId job_id, JobEvent event);
    void record_block_exec_time(unsigned long long start, unsigned long long end);
    // one kernel's placement prediction against what its workgroups reported: workgroups, mispredicted workgroups,
    // compute units they had been predicted on (reference src/server/profiler.cpp:146-150, file format :93-97)
    void record_kernel_block_mis_alloc(unsigned total, unsigned total_wrong_prediction, unsigned total_wrong_prediction_cus);
    // the reference's spelling of the same call
    void recrod_kernel_block_mis_alloc(unsigned total, unsigned wrong, unsigned wrong_sm) { record_kernel_block_mis_alloc(total, wrong, wrong_sm); }
    bool recording_run_next_times() const { return run_next_times_flag_; }
    void record_run_next_time(TimePoint start, TimePoint end, unsigned num_blocks);
    // num workgroups of the job's running stage acquired or released (reference src/server/sm_resources.cpp:48,64)
    void record_resource_event(job::Job* job, unsigned num, ResourceEvent event);
    // the job's next stage has joined the ready queue (reference src/server/scheduler_full3.cpp:175,244,304)
    void record_queued_resource_event(job::Job* job);

  private:
    ipc::ShmChannelCpuReader* c2s_channel_;
    bool kernel_info_flag_ = false;
    bool job_events_flag_ = false;
    bool run_next_times_flag_ = false;
    bool resource_events_flag_ = false;
    bool block_exec_times_flag_ = false;
    bool mis_alloc_flag_ = false;
    std::vector<std::tuple<unsigned, unsigned, unsigned>> mis_alloc_;
    std::vector<std::pair<unsigned long long, unsigned long long>> block_exec_times_;
    std::vector<std::tuple<TimePoint, TimePoint, unsigned>> run_next_times_;
    std::vector<std::tuple<JobId, std::string, ResourceEvent, TimePoint, unsigned, unsigned, unsigned, unsigned>> resource_events_;
    std::vector<std::tuple<TimePoint, TimePoint, unsigned, unsigned, unsigned, unsigned, double, unsigned>> kernel_info_;
    std::vector<std::vector<std::pair<JobEvent, TimePoint>>> jobs_events_cur_;
    std::vector<std::vector<std::pair<JobEvent, TimePoint>>> jobs_events_all_;
};

}  // namespace server
}  // namespace llis
