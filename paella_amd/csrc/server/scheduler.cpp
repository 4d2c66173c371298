#include <llis/job/context.h>
#include <llis/server/phase_clock.h>
#include <llis/server/scheduler.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <stdexcept>

namespace llis {
namespace server {

// ------------------------------------------------------------------------------------------ factory

std::unordered_map<std::string, SchedulerFactory::RegisterFunc>& SchedulerFactory::registry() {
    static std::unordered_map<std::string, RegisterFunc> map;  // built on first use: safe from static initialisers
    return map;
}

bool SchedulerFactory::register_scheduler(std::string name, RegisterFunc func) { return registry().emplace(std::move(name), std::move(func)).second; }

std::unique_ptr<Scheduler> SchedulerFactory::create(std::string name, const SchedulerOptions& options) {
    auto it = registry().find(name);
    if (it == registry().end()) {
        std::string known;
        for (const auto& n : names()) known += " " + n;
        throw std::invalid_argument("unknown scheduler '" + name + "'; available:" + known);
    }
    return it->second(options);
}

std::vector<std::string> SchedulerFactory::names() {
    std::vector<std::string> out;
    for (const auto& kv : registry()) out.push_back(kv.first);
    return out;
}

// ------------------------------------------------------------------------------------------ shared plumbing

StreamPoolScheduler::StreamPoolScheduler(const SchedulerOptions& options, size_t mem2sched_bytes)
    : options_(options), gpu2sched_channel_(options.ring_slots), mem2sched_channel_(mem2sched_bytes) {
    job::Context::set_gpu2sched_channel(&gpu2sched_channel_);
    job::Context::set_mem2sched_channel(&mem2sched_channel_);

    streams_.resize(options.num_streams);
    for (unsigned i = 0; i < options.num_streams; ++i) {
        LLIS_CHECK_HIP(llis_hip_stream_create(&streams_[i]));
        stream_index_[streams_[i]] = i;
        free_streams_.push_back(i);
    }
    if (options.measure_block_time) gpu2sched_block_time_channel_.connect(std::string(), options.ring_slots);
    job::Context::set_gpu2sched_block_time_channel(options.measure_block_time ? &gpu2sched_block_time_channel_ : nullptr);
    notifiers_raw_ = job::FinishedBlockNotifier::create_array(options.num_streams, &gpu2sched_channel_,
                                                              options.measure_block_time ? &gpu2sched_block_time_channel_ : nullptr,
                                                              options.noti_batch ? options.noti_batch : job::FinishedBlockNotifier::noti_batch_size);
    for (unsigned i = 0; i < options.num_streams; ++i) free_notifiers_.push_back(i);
}

StreamPoolScheduler::~StreamPoolScheduler() {
    LLIS_WARN_HIP(llis_hip_device_synchronize());
    for (void* s : streams_) LLIS_WARN_HIP(llis_hip_stream_destroy(s));
    job::FinishedBlockNotifier::free_array(notifiers_raw_);
}

void StreamPoolScheduler::try_handle_block_start_finish() {
    if (gpu2sched_channel_.can_read<job::InstrumentInfo>()) {
        LLIS_PHASE(kRing);
        const job::InstrumentInfo info = gpu2sched_channel_.read<job::InstrumentInfo>();
        job::Job* job = job_of(info.job_id);
        cur_smid_ = info.smid;
        // the compute unit goes into the log only where the scheduler reads it
        const int64_t logged_cu = options_.per_cu_placement && job->reports_cu() ? (int64_t)info.smid : -1;
        if (info.is_start == 1) {
            log_->add('B', info.job_id, 1, info.num, logged_cu);
            handle_block_start(job, info.num);
        } else if (info.is_start == 0) {
            log_->add('B', info.job_id, 0, info.num, logged_cu);
            handle_block_finish(job, info.num);
        } else {
            log_->add('M', info.job_id);
            handle_mem_finish(job);
        }
    }
    else {
        LLIS_PHASE(kIdle);
    }
    while (options_.measure_block_time && gpu2sched_block_time_channel_.can_read<job::BlockStartEndTime>()) {
        // unpacking as in reference src/server/scheduler_full3.cpp:113-119
        const job::BlockStartEndTime t = gpu2sched_block_time_channel_.read<job::BlockStartEndTime>();
        const uint32_t start = (uint32_t)t.data[0] << 8 | (uint32_t)(t.data[1] >> 8);
        const uint32_t end = (uint32_t)(t.data[1] & 0xFF) << 16 | t.data[2];
        profiler_->record_block_exec_time(start, end);
    }
    if (mem2sched_channel_.can_read()) {
        LLIS_PHASE(kRing);
        job::Job* job;
        mem2sched_channel_.read(&job);
        log_->add('M', job->get_id());
        handle_mem_finish(job);
    }
}

job::Job* StreamPoolScheduler::adopt(std::unique_ptr<job::Job> owned) {
    job::Job* job = owned.get();
    if (unused_job_id_.empty()) {
        job->set_id((JobId)job_id_to_job_map_.size());
        job_id_to_job_map_.push_back(std::move(owned));
    } else {
        job->set_id(unused_job_id_.back());
        unused_job_id_.pop_back();
        job_id_to_job_map_[job->get_id()] = std::move(owned);
    }
    return job;
}

void StreamPoolScheduler::retire(job::Job* job) {
    const JobId id = job->get_id();
    unused_job_id_.push_back(id);
    server_->release_job_instance(std::move(job_id_to_job_map_[id]));
}

void StreamPoolScheduler::give_stream(job::Job* job) { free_streams_.push_back(stream_index_.at(reinterpret_cast<void*>(job->get_cuda_stream()))); }

void StreamPoolScheduler::give_notifier(job::Job* job) { free_notifiers_.push_back((unsigned)(job->get_finished_block_notifier() - notifiers_raw_)); }

void StreamPoolScheduler::post_mem_completion(job::Job* job) {
    void* stream = reinterpret_cast<void*>(job->get_cuda_stream());
    if (options_.mem_marker) {
        job::InstrumentInfo info;
        info.is_start = 2;
        info.num = 1;
        info.job_id = job->get_id();
        uint64_t bits;
        __builtin_memcpy(&bits, &info, sizeof(bits));
        LLIS_CHECK_HIP(llis_hip_launch_ring_marker(stream, gpu2sched_channel_.get_slots(), (unsigned)gpu2sched_channel_.get_count(),
                                                   gpu2sched_channel_.get_cursor(), bits));
    } else {
        LLIS_CHECK_HIP(llis_hip_launch_host_func(stream, &StreamPoolScheduler::mem_notification_callback, job));
    }
}

void StreamPoolScheduler::mem_notification_callback(void* job) {
    // Runs on a runtime thread; several streams may complete at once, so serialise whole messages.
    job::Context::post_mem_completion(static_cast<job::Job*>(job));
}

void StreamPoolScheduler::spin_sleep() const {
    for (volatile unsigned i = 0; i < options_.sched_sleep; ++i) {
    }
}

}  // namespace server
}  // namespace llis
