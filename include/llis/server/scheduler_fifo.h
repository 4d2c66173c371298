#pragma once
// "fifo": job-by-job dispatch.  A job taken from the arrival queue gets one stream and one notifier and
// ALL of its stages are issued back to back on that stream; the scheduler then only counts completed
// workgroups (a copy stage counts as one) to know when to wake the client (all work up to and including
// the pre-notify stage has finished) and when the job is done.  With one stream this is single-stream
// serving, with many it is plain multi-stream serving
// (reference include/llis/server/scheduler_fifo.h, src/server/scheduler_fifo.cpp:26-268).

#include <llis/server/scheduler.h>

#include <deque>

namespace llis {
namespace server {

class SchedulerFifo : public StreamPoolScheduler {
  public:
    explicit SchedulerFifo(const SchedulerOptions& options);
    void handle_new_job(std::unique_ptr<job::Job> job) override;

  protected:
    void handle_block_start(job::Job*, unsigned) override {}
    void handle_block_finish(job::Job* job, unsigned num) override { account_finished(job, (int)num); }
    void handle_mem_finish(job::Job* job) override { account_finished(job, 1); }

  private:
    struct Progress {
        unsigned remaining_blocks = 0;
        int pre_notify_blocks = 0;
        bool pre_notify_sent = false;
    };

    void account_finished(job::Job* job, int num);
    void schedule_job();

    std::deque<job::Job*> job_queue_;
    std::vector<Progress> progress_;  // indexed by JobId
};

}  // namespace server
}  // namespace llis
