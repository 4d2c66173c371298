#include <llis/job/context.h>
#include <llis/server/phase_clock.h>
#include <llis/server/scheduler_full3.h>

#include <chrono>

namespace llis {
namespace server {

// ------------------------------------------------------------------------------------------ JobQueue

void JobQueue::push(job::Job* job) {
    const unsigned type_id = job->get_registered_job_id();
    if (type_id >= types_.size()) types_.resize(type_id + 1);
    TypeState& ts = types_[type_id];
    if (!ts.known) {  // a type that is new, or whose queue ran dry, starts from the current baseline
        ts.known = true;
        ts.deficit = new_type_deficit_;
        ++num_types_;
    }
    if (ts.jobs.empty()) {
        ts.seq = next_seq_++;
        active_types_.insert(TypeKey{ts.deficit, ts.seq, type_id});
    }
    const JobKey key{job->get_priority(), next_seq_++, job};
    all_.insert(key);
    ts.jobs.insert(key);
}

const JobQueue::JobKey& JobQueue::select(unsigned* type_id) const {
    const TypeKey& starved = *active_types_.begin();
    if (starved.deficit >= unfairness_threshold_) {
        *type_id = starved.type_id;
        return *types_[starved.type_id].jobs.begin();
    }
    const JobKey& best = *all_.begin();
    *type_id = best.job->get_registered_job_id();
    return best;
}

job::Job* JobQueue::top() {
    unsigned type_id;
    return select(&type_id).job;
}

job::Job* JobQueue::pop() {
    unsigned type_id;
    const JobKey key = select(&type_id);
    TypeState& ts = types_[type_id];
    all_.erase(key);
    ts.jobs.erase(key);

    // Everybody's entitlement grows by one fair share; expressed by lowering the baseline and the threshold.
    const double fair_share = 1. / (double)num_types_;
    new_type_deficit_ -= fair_share;
    unfairness_threshold_ -= fair_share;

    active_types_.erase(TypeKey{ts.deficit, ts.seq, type_id});
    if (ts.jobs.empty()) {
        ts.known = false;  // forget the type's history once nothing of it is queued
        --num_types_;
    } else {
        ts.deficit -= 1.;  // the served type pays for the dispatch
        ts.seq = next_seq_++;
        active_types_.insert(TypeKey{ts.deficit, ts.seq, type_id});
    }
    return key.job;
}

// ------------------------------------------------------------------------------------------ SchedulerFull3

SchedulerFull3::SchedulerFull3(const SchedulerOptions& options) : StreamPoolScheduler(options, 409600), job_queue_(options.unfair) {
    job::Context::set_stage_by_stage(true);
    if (options.per_cu_placement) per_cu_ = std::make_unique<GpuResources>();
}

SchedulerFull3::SchedulerFull3(const SchedulerOptions& options, std::unique_ptr<GpuResources> per_cu)
    : StreamPoolScheduler(options, 409600), job_queue_(options.unfair), per_cu_(std::move(per_cu)) {
    job::Context::set_stage_by_stage(true);
    options_.per_cu_placement = true;
}

SchedulerFull3::SchedulerFull3(const SchedulerOptions& options, const SmResources& budget)
    : StreamPoolScheduler(options, 409600), job_queue_(options.unfair), gpu_resources_(budget) {
    job::Context::set_stage_by_stage(true);
}

void SchedulerFull3::set_server(Server* server) {
    Scheduler::set_server(server);
    gpu_resources_.set_profiler(profiler_);
    if (per_cu_) per_cu_->set_profiler(profiler_);
}

double SchedulerFull3::take_priority(job::Job* job) const {
    const double remaining = job->get_cur_rl();
    job->dec_cur_rl();  // the stage being queued no longer counts as "remaining" next time
    return -remaining;
}

void SchedulerFull3::handle_new_job(std::unique_ptr<job::Job> owned) {
    if (!owned->has_next()) {
        server_->release_job_instance(std::move(owned));
        return;
    }
    const bool first_is_mem = owned->is_mem();
    job::Job* job = adopt(std::move(owned));
    log_->add('J', job->get_id(), job->get_registered_job_id(), job->get_unique_id(), first_is_mem);
    profiler_->record_job_event(job->get_id(), Profiler::JobEvent::JOB_SUBMITTED);

    const unsigned next_stage = (unsigned)(job->get_cur_stage() + 1);
    if (!server_->has_job_stage_resource(job, next_stage)) server_->set_job_stage_resource(job, next_stage, 1);
    job->set_stage_lengths_resources(server_->get_job_remaining_rl(job, 0), server_->get_job_stage_lengths(job), server_->get_job_stage_resources(job));
    job->set_priority(take_priority(job));
    if (!job->is_mem()) profiler_->record_queued_resource_event(job);

    job_queue_.push(job);
    ++num_jobs_;
    schedule_job();
}

void SchedulerFull3::handle_block_start(job::Job* job, unsigned num) {
    const bool names_cu = per_cu_ && job->reports_cu();
    if (names_cu) per_cu_->observe_block_start(job, cur_smid_);
    if (job->mark_block_start(num)) return;  // some workgroups still waiting for a CU
    if (names_cu) {
        // every workgroup has said where it runs: predictions that did not come true are given back
        unsigned wrong_cus = 0;
        const unsigned wrong = per_cu_->reconcile(job, &wrong_cus);
        log_->add('R', job->get_id(), wrong, wrong_cus);
    }
    if (job->is_unfit()) {
        // The over-subscribed kernel is now fully resident: its credit returns and the queue may move.
        job->unset_unfit();
        --num_outstanding_kernels_;
        schedule_job();
    }
}

void SchedulerFull3::requeue_or_finish(job::Job* job) {
    const auto end_time = std::chrono::steady_clock::now();
    const double length = std::chrono::duration<double, std::micro>(end_time - job->get_stage_start_time()).count();
    log_->add('L', job->get_id(), job->get_cur_stage(), 0, 0, 0, length);
    server_->update_job_stage_length(job, (unsigned)job->get_cur_stage(), length);

    if (job->has_next()) {
        const unsigned next_stage = (unsigned)(job->get_cur_stage() + 1);
        if (!server_->has_job_stage_resource(job, next_stage)) server_->set_job_stage_resource(job, next_stage, 1);
        job->set_priority(take_priority(job));
        if (!job->is_mem()) profiler_->record_queued_resource_event(job);
        job_queue_.push(job);
    } else {
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::JOB_FINISHED);
        log_->add('E', job->get_id());
        server_->notify_job_ends(job);
        --num_jobs_;
    }
}

void SchedulerFull3::handle_block_finish(job::Job* job, unsigned num) {
    job->mark_block_finish(num);
    const bool stage_over = !job->is_running();
    if (stage_over) {
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_FINISHED);
        profiler_->record_kernel_info(job->get_stage_start_time(), std::chrono::steady_clock::now(), job->get_cur_num_blocks(),
                                      job->get_cur_num_threads_per_block(), job->get_cur_smem_size_per_block(),
                                      job->get_cur_num_registers_per_thread(), job->get_priority(), job->get_registered_job_id());
        requeue_or_finish(job);
        if (job->is_unfit()) {  // finished before its start messages were all seen
            job->unset_unfit();
            --num_outstanding_kernels_;
        }
        give_stream(job);
        give_notifier(job);
    }
    if (!per_cu_) gpu_resources_.release(job, (int)num);
    else if (job->reports_cu()) per_cu_->observe_block_finish(job, cur_smid_);
    else per_cu_->release_predicted(job, num);
    if (stage_over && !job->has_next()) retire(job);
    schedule_job();
}

void SchedulerFull3::handle_mem_finish(job::Job* job) {
    job->unset_running();
    requeue_or_finish(job);
    give_stream(job);
    if (!job->has_next()) retire(job);
    schedule_job();
}

void SchedulerFull3::schedule_job() {
    while (has_stream() && !job_queue_.empty()) {
        job::Job* job = job_queue_.top();
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SCHED_START);
        spin_sleep();

        const bool is_mem = job->is_mem();
        const bool posts_itself = is_mem && job->completes_itself();  // read before run_next declares the stage after
        bool unfit = false;
        if (!is_mem && !(per_cu_ ? per_cu_->job_fits(job) : gpu_resources_.job_fits(job))) {
            if (num_outstanding_kernels_ >= (int)options_.extra_kernels) {
                profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SCHED_ABORT);
                break;  // head-of-queue blocking is intended: nothing overtakes the best job
            }
            ++num_outstanding_kernels_;
            job->set_unfit();
            unfit = true;
        }
        job_queue_.pop();
        if (!job->has_started()) job->set_started();

        const unsigned stream = take_stream();
        job->set_running(stream_handle(stream));
        long long notifier = -1;
        if (!is_mem) {
            notifier = take_notifier();
            job->set_finished_block_notifier(notifier_ptr((unsigned)notifier));
            if (per_cu_) per_cu_->choose_cus(job);
            else gpu_resources_.acquire(job, (int)job->get_cur_num_blocks());
        }
        log_->add('D', job->get_id(), job->get_cur_stage(), stream, notifier, is_mem, unfit);
        if (job->is_pre_notify()) {
            log_->add('S', job->get_id());
            server_->notify_job_starts(job);
        }

        job::Context::set_current_job(job);
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SUBMIT_START);
        {
            LLIS_PHASE_IF(is_mem, kLaunchCopy, kLaunch);
            if (profiler_->recording_run_next_times()) {
                const auto t0 = std::chrono::steady_clock::now();
                job->run_next();
                profiler_->record_run_next_time(t0, std::chrono::steady_clock::now(), job->get_cur_num_blocks());
            } else {
                job->run_next();
            }
            if (is_mem && !posts_itself) post_mem_completion(job);
            // a kernel stage that did not ask for its notifier reports through the un-aggregated hooks
            if (per_cu_) job->set_reports_cu(!is_mem && !job->used_finished_block_notifier());
        }
        profiler_->record_job_event(job->get_id(), Profiler::JobEvent::KERNEL_SUBMIT_END);
    }
}

LLIS_SCHEDULER_REGISTER("full3", [](const SchedulerOptions& o) -> std::unique_ptr<Scheduler> { return std::make_unique<SchedulerFull3>(o); });

}  // namespace server
}  // namespace llis
