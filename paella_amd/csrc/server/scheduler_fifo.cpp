#include <llis/job/context.h>
#include <llis/server/scheduler_fifo.h>

namespace llis {
namespace server {

SchedulerFifo::SchedulerFifo(const SchedulerOptions& options) : StreamPoolScheduler(options, 10240) { job::Context::set_stage_by_stage(false); }

void SchedulerFifo::handle_new_job(std::unique_ptr<job::Job> owned) {
    if (!owned->has_next()) {  // a job without stages has nothing to run
        server_->release_job_instance(std::move(owned));
        return;
    }
    const bool first_is_mem = owned->is_mem();
    job::Job* job = adopt(std::move(owned));
    if (progress_.size() <= job->get_id()) progress_.resize(job->get_id() + 1);
    progress_[job->get_id()] = Progress();
    log_->add('J', job->get_id(), job->get_registered_job_id(), job->get_unique_id(), first_is_mem);
    job_queue_.push_back(job);
    ++num_jobs_;
    schedule_job();
}

void SchedulerFifo::account_finished(job::Job* job, int num) {
    Progress& pr = progress_[job->get_id()];
    pr.remaining_blocks -= (unsigned)num;
    pr.pre_notify_blocks -= num;
    if (pr.pre_notify_blocks <= 0 && !pr.pre_notify_sent) {
        log_->add('S', job->get_id());
        server_->notify_job_starts(job);
        pr.pre_notify_sent = true;
    }
    if (pr.remaining_blocks == 0) {
        log_->add('E', job->get_id());
        server_->notify_job_ends(job);
        give_stream(job);
        give_notifier(job);
        retire(job);
        --num_jobs_;
    }
    schedule_job();
}

void SchedulerFifo::schedule_job() {
    while (has_stream() && !job_queue_.empty()) {
        job::Job* job = job_queue_.front();
        job_queue_.pop_front();

        job->set_started();
        const unsigned stream = take_stream();
        const unsigned notifier = take_notifier();
        job->set_running(stream_handle(stream));
        job->set_finished_block_notifier(notifier_ptr(notifier));
        job::Context::set_current_job(job);

        Progress& pr = progress_[job->get_id()];
        bool saw_pre_notify = false;
        int stage = 0;
        while (job->has_next()) {
            const bool is_mem = job->is_mem();
            const unsigned units = is_mem ? 1u : job->get_num_blocks();
            pr.remaining_blocks += units;
            if (!saw_pre_notify) {
                pr.pre_notify_blocks += (int)units;
                if (job->is_pre_notify()) saw_pre_notify = true;
            }
            log_->add('D', job->get_id(), stage++, stream, notifier, is_mem, 0);
            job->run_next();
            if (is_mem) post_mem_completion(job);
        }
    }
}

LLIS_SCHEDULER_REGISTER("fifo", [](const SchedulerOptions& o) -> std::unique_ptr<Scheduler> { return std::make_unique<SchedulerFifo>(o); });

}  // namespace server
}  // namespace llis
