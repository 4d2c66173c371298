#pragma once
// "fifo2": kernel-by-kernel dispatch in arrival order.  Every stage is issued separately on whatever
// stream is free; among jobs with a pending stage the one that arrived first (smallest unique id) goes
// next.  No occupancy model, no priorities
// (reference include/llis/server/scheduler_fifo2.h:33-62, src/server/scheduler_fifo2.cpp:23-269).

#include <llis/server/scheduler.h>

#include <queue>

namespace llis {
namespace server {

class SchedulerFifo2 : public StreamPoolScheduler {
  public:
    explicit SchedulerFifo2(const SchedulerOptions& options);
    void handle_new_job(std::unique_ptr<job::Job> job) override;

  protected:
    void handle_block_start(job::Job*, unsigned) override {}
    void handle_block_finish(job::Job* job, unsigned num) override;
    void handle_mem_finish(job::Job* job) override;

  private:
    struct ArrivedLater {
        bool operator()(const job::Job* a, const job::Job* b) const { return a->get_unique_id() > b->get_unique_id(); }
    };

    void stage_done(job::Job* job, bool was_kernel);
    void schedule_job();

    std::priority_queue<job::Job*, std::vector<job::Job*>, ArrivedLater> job_queue_;
};

}  // namespace server
}  // namespace llis
