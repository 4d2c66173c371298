#include <llis/server/profiler.h>

#include <cstdio>
#include <typeinfo>

namespace llis {
namespace server {

void Profiler::handle_cmd() {
    ProfilerMsgType sub;
    c2s_channel_->read(&sub);
    const unsigned v = (unsigned)sub;
    if (sub == ProfilerMsgType::SAVE) {
        std::string prefix;
        c2s_channel_->read(&prefix);
        save(prefix);
        return;
    }
    const bool on = (v % 2) == 0;  // SET_* are even, UNSET_* odd
    switch (v / 2) {
        case 0: kernel_info_flag_ = on; break;
        case 4: job_events_flag_ = on; break;
        case 1: block_exec_times_flag_ = on; break;
        case 2: mis_alloc_flag_ = on; break;
        case 3: run_next_times_flag_ = on; break;
        case 5: resource_events_flag_ = on; break;
        default: std::fprintf(stderr, "[llis] unknown profiler command %u ignored\n", v); break;
    }
}

void Profiler::record_kernel_info(TimePoint start, TimePoint end, unsigned num_blocks, unsigned num_threads_per_block, unsigned smem_size_per_block,
                                  unsigned num_registers_per_thread, double priority, unsigned job_ref_id) {
    if (kernel_info_flag_) kernel_info_.emplace_back(start, end, num_blocks, num_threads_per_block, smem_size_per_block, num_registers_per_thread, priority, job_ref_id);
}

void Profiler::record_job_event(JobId job_id, JobEvent event) {
    if (!job_events_flag_) return;
    if (jobs_events_cur_.size() <= job_id) jobs_events_cur_.resize(job_id + 1);
    auto& cur = jobs_events_cur_[job_id];
    if (event == JobEvent::JOB_SUBMITTED) cur.clear();
    cur.emplace_back(event, std::chrono::steady_clock::now());
    if (event == JobEvent::JOB_FINISHED) {
        jobs_events_all_.push_back(std::move(cur));
        cur.clear();
    }
}

void Profiler::record_block_exec_time(unsigned long long start, unsigned long long end) {
    if (block_exec_times_flag_) block_exec_times_.emplace_back(start, end);
}

void Profiler::record_kernel_block_mis_alloc(unsigned total, unsigned total_wrong_prediction, unsigned total_wrong_prediction_cus) {
    if (mis_alloc_flag_) mis_alloc_.emplace_back(total, total_wrong_prediction, total_wrong_prediction_cus);
}

void Profiler::record_run_next_time(TimePoint start, TimePoint end, unsigned num_blocks) {
    if (run_next_times_flag_) run_next_times_.emplace_back(start, end, num_blocks);
}

void Profiler::record_resource_event(job::Job* job, unsigned num, ResourceEvent event) {
    if (!resource_events_flag_) return;
    resource_events_.emplace_back(job->get_unique_id(), typeid(*job).name(), event, std::chrono::steady_clock::now(), num, job->get_cur_num_threads_per_block(),
                                  job->get_cur_smem_size_per_block(), job->get_cur_num_registers_per_thread());
}

void Profiler::record_queued_resource_event(job::Job* job) {
    if (!resource_events_flag_) return;
    resource_events_.emplace_back(job->get_unique_id(), typeid(*job).name(), ResourceEvent::QUEUED, std::chrono::steady_clock::now(), job->get_num_blocks(),
                                  job->get_num_threads_per_block(), job->get_smem_size_per_block(), job->get_num_registers_per_thread());
}

void Profiler::save(const std::string& prefix) {
    auto ns = [](TimePoint t) { return (long long)t.time_since_epoch().count(); };
    if (FILE* fp = std::fopen((prefix + "_kernel_info.txt").c_str(), "w")) {
        for (const auto& k : kernel_info_)
            std::fprintf(fp, "%lld %lld %u %u %u %u %f %u\n", ns(std::get<0>(k)), ns(std::get<1>(k)), std::get<2>(k), std::get<3>(k), std::get<4>(k),
                         std::get<5>(k), std::get<6>(k), std::get<7>(k));
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((prefix + "_job_events.txt").c_str(), "w")) {
        for (const auto& job : jobs_events_all_) {
            for (const auto& ev : job)
                std::fprintf(fp, "%u %f ", (unsigned)ev.first, std::chrono::duration<double, std::micro>(ev.second.time_since_epoch()).count());
            std::fprintf(fp, "\n");
        }
        std::fclose(fp);
    }
    auto us = [](TimePoint t) { return std::chrono::duration<double, std::micro>(t.time_since_epoch()).count(); };
    if (FILE* fp = std::fopen((prefix + "_run_next_times.txt").c_str(), "w")) {
        for (const auto& r : run_next_times_)
            std::fprintf(fp, "%f %f %f %u\n", us(std::get<0>(r)), us(std::get<1>(r)),
                         std::chrono::duration<double, std::micro>(std::get<1>(r) - std::get<0>(r)).count(), std::get<2>(r));
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((prefix + "_resource_events.txt").c_str(), "w")) {
        for (const auto& r : resource_events_)
            std::fprintf(fp, "%u %s %u %f %u %u %u %u\n", (unsigned)std::get<0>(r), std::get<1>(r).c_str(), (unsigned)std::get<2>(r), us(std::get<3>(r)), std::get<4>(r),
                         std::get<5>(r), std::get<6>(r), std::get<7>(r));
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((prefix + "_block_exec_times.txt").c_str(), "w")) {
        for (const auto& b : block_exec_times_) std::fprintf(fp, "%llu %llu\n", b.first, b.second);
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((prefix + "_kernel_block_mis_alloc.txt").c_str(), "w")) {
        for (const auto& m : mis_alloc_) std::fprintf(fp, "%u %u %u\n", std::get<0>(m), std::get<1>(m), std::get<2>(m));
        std::fclose(fp);
    }
    mis_alloc_.clear();
    kernel_info_.clear();
    jobs_events_all_.clear();
    run_next_times_.clear();
    block_exec_times_.clear();
    resource_events_.clear();
}

}  // namespace server
}  // namespace llis
