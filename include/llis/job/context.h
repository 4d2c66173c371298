#pragma once
// Process-wide state shared by the server, the job definitions it loads and the kernel library: the job
// whose stage is being issued right now, and non-owning endpoints of the two completion channels
// (workgroup messages from the GPU, copy-stage completions from runtime callback threads).
// One definition lives in libllis_core.so so every loaded job sees the same copy
// (reference include/llis/job/context.h:10-53, src/job/context.cpp:8-13).

#include <llis/ipc/shm_channel.h>
#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/job.h>

namespace llis {
namespace job {

class Context {
  public:
    static Job* get_current_job() { return current_job_; }
    static void set_current_job(Job* job) { current_job_ = job; }

    static void set_gpu2sched_channel(ipc::Gpu2SchedChannel* channel) { gpu2sched_channel_ = channel->fork(); }
    static ipc::Gpu2SchedChannel* get_gpu2sched_channel() { return &gpu2sched_channel_; }

    // nullptr: the active scheduler collects no per-workgroup timing (a handle left by an earlier scheduler of
    // this process must not survive it)
    static void set_gpu2sched_block_time_channel(ipc::Gpu2SchedChannel* channel) {
        gpu2sched_block_time_channel_ = channel ? channel->fork() : ipc::Gpu2SchedChannel();
    }
    static ipc::Gpu2SchedChannel* get_gpu2sched_block_time_channel() { return &gpu2sched_block_time_channel_; }

    static void set_mem2sched_channel(ipc::ShmChannelCpuReader* channel) { mem2sched_channel_ = channel->fork(); }
    static ipc::ShmChannelCpuWriter* get_mem2sched_channel() { return &mem2sched_channel_; }
    // Tells the scheduler that the job's copy stage is over (what its own marker or host callback would have told it); for
    // stages declared with Job::set_completes_itself().  Callable from any thread.  Not in the reference.
    static void post_mem_completion(Job* job) {
        mem2sched_channel_.acquire_writer_lock();
        mem2sched_channel_.write(job);
        mem2sched_channel_.release_writer_lock();
    }

    // True when the active scheduler issues a job's next stage only after the previous one has been reported
    // finished (fifo2, full3); false when it issues all stages at once and relies on stream order (fifo).
    // A job may submit its kernels outside its stream only in the first case.  Not in the reference, whose
    // jobs always launch on the stream.
    static void set_stage_by_stage(bool v) { stage_by_stage_ = v; }
    static bool is_stage_by_stage() { return stage_by_stage_; }

    // Functions the serving thread calls once per turn of its loop, after it has looked at its rings: for job libraries
    // that hold work back and release it from that thread (a function is added once, however often it is registered).
    // Not in the reference.
    using PollHook = void (*)();
    static void add_poll_hook(PollHook fn);
    static void run_poll_hooks() {
        for (unsigned i = 0; i < num_poll_hooks_; ++i) poll_hooks_[i]();
    }

  private:
    static constexpr unsigned kMaxPollHooks = 8;
    static PollHook poll_hooks_[kMaxPollHooks];
    static unsigned num_poll_hooks_;
    static bool stage_by_stage_;
    static Job* current_job_;
    static ipc::Gpu2SchedChannel gpu2sched_channel_;
    static ipc::Gpu2SchedChannel gpu2sched_block_time_channel_;
    static ipc::ShmChannelCpuWriter mem2sched_channel_;
};

}  // namespace job
}  // namespace llis
