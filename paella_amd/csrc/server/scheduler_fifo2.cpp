#include <llis/job/context.h>
#include <llis/server/scheduler_fifo2.h>

namespace llis {
namespace server {

SchedulerFifo2::SchedulerFifo2(const SchedulerOptions& options) : StreamPoolScheduler(options, 10240) { job::Context::set_stage_by_stage(true); }

void SchedulerFifo2::handle_new_job(std::unique_ptr<job::Job> owned) {
    if (!owned->has_next()) {
        server_->release_job_instance(std::move(owned));
        return;
    }
    const bool first_is_mem = owned->is_mem();
    job::Job* job = adopt(std::move(owned));
    log_->add('J', job->get_id(), job->get_registered_job_id(), job->get_unique_id(), first_is_mem);
    profiler_->record_job_event(job->get_id(), Profiler::JobEvent::JOB_SUBMITTED);
    job_queue_.push(job);
    ++num_jobs_;
    schedule_job();
}

void SchedulerFifo2::stage_done(job::Job* job, bool was_kernel) {
    profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_FINISHED);
    const bool more = job->has_next();
    if (more) {
        job_queue_.push(job);
    } else {
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::JOB_FINISHED);
        log_->add('E', job->get_id());
        server_->notify_job_ends(job);
        --num_jobs_;
    }
    give_stream(job);
    if (was_kernel) give_notifier(job);
    if (!more) retire(job);
}

void SchedulerFifo2::handle_block_finish(job::Job* job, unsigned num) {
    job->mark_block_finish(num);
    if (!job->is_running()) stage_done(job, true);
    schedule_job();
}

void SchedulerFifo2::handle_mem_finish(job::Job* job) {
    job->unset_running();
    stage_done(job, false);
    schedule_job();
}

void SchedulerFifo2::schedule_job() {
    while (has_stream() && !job_queue_.empty()) {
        job::Job* job = job_queue_.top();
        job_queue_.pop();
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SCHED_START);
        if (!job->has_started()) job->set_started();

        const unsigned stream = take_stream();
        job->set_running(stream_handle(stream));
        const bool is_mem = job->is_mem();
        const bool posts_itself = is_mem && job->completes_itself();  // read before run_next declares the stage after
        long long notifier = -1;
        if (!is_mem) {
            notifier = take_notifier();
            job->set_finished_block_notifier(notifier_ptr((unsigned)notifier));
        }
        log_->add('D', job->get_id(), job->get_cur_stage(), stream, notifier, is_mem, 0);
        if (job->is_pre_notify()) {
            log_->add('S', job->get_id());
            server_->notify_job_starts(job);
        }
        job::Context::set_current_job(job);
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SUBMIT_START);
        if (profiler_->recording_run_next_times()) {
            const auto t0 = std::chrono::steady_clock::now();
            job->run_next();
            profiler_->record_run_next_time(t0, std::chrono::steady_clock::now(), is_mem ? 0 : job->get_cur_num_blocks());
        } else {
            job->run_next();
        }
        if (is_mem && !posts_itself) post_mem_completion(job);
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SUBMIT_END);
    }
}

LLIS_SCHEDULER_REGISTER("fifo2", [](const SchedulerOptions& o) -> std::unique_ptr<Scheduler> { return std::make_unique<SchedulerFifo2>(o); });

}  // namespace server
}  // namespace llis
