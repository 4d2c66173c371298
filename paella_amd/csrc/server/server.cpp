#include <llis/job/context.h>
#include <llis/ipc/name_format.h>
#include <llis/server/scheduler.h>
#include <llis/server/server.h>
#include <llis/server/phase_clock.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>

namespace llis {
namespace server {

Server::Server(std::string server_name, Scheduler* scheduler)
    : server_name_(std::move(server_name)),
      scheduler_(scheduler),
      c2s_channel_(ipc::c2s_channel_name(server_name_), c2s_channel_size),
      profiler_(&c2s_channel_) {
    if (const char* path = std::getenv("LLIS_EVENT_LOG")) {
        if (*path) event_log_.enable(true);
    }
    if (const char* skip = std::getenv("LLIS_IPC_LATENCY_SKIP")) ipc_latency_skip_ = (unsigned)std::strtoul(skip, nullptr, 10);
    scheduler_->set_server(this);
}

Server::~Server() {
    if (ipc_latency_count_) {
        std::printf("Avg launch job IPC latency: %f us over %llu requests\n", ipc_latency_mean_us(), (unsigned long long)ipc_latency_count_);
        std::fflush(stdout);
    }
    LLIS_PHASE_REPORT();
    if (const char* path = std::getenv("LLIS_EVENT_LOG")) {
        if (*path && event_log_.enabled()) event_log_.save(path);
    }
}

void Server::serve() {
    while (!stop_.load(std::memory_order_acquire)) poll_once();
}

void Server::poll_once() {
    if (c2s_channel_.can_read()) {
        LLIS_PHASE(kRequests);
        handle_c2s();
    }
    scheduler_->try_handle_block_start_finish();
    {
        LLIS_PHASE(kHooks);
        job::Context::run_poll_hooks();
    }
    if (total_owed_wakeups_ != 0 && ++polls_since_retry_ >= 64) retry_owed_wakeups();
}

void Server::retry_owed_wakeups() {
    polls_since_retry_ = 0;
    for (auto& conn : client_connections_) total_owed_wakeups_ -= conn->retry_wakeups();
}

void Server::handle_c2s() {
    MsgType type;
    c2s_channel_.read(&type);
    switch (type) {
        case MsgType::REGISTER_CLIENT: handle_register_client(); break;
        case MsgType::REGISTER_JOB: handle_register_job(); break;
        case MsgType::LAUNCH_JOB: handle_launch_job(); break;
        case MsgType::GROW_POOL: handle_grow_pool(); break;
        case MsgType::CUDA_PROFILER_START: LLIS_WARN_HIP(llis_hip_profiler_start()); break;
        case MsgType::CUDA_PROFILER_STOP: LLIS_WARN_HIP(llis_hip_profiler_stop()); break;
        case MsgType::PROFILER_CMD:
            // A recording covers whole jobs.  A job whose client was woken when its last stage was dispatched (pre-notify) may
            // still have that kernel running when the client's next message arrives: the switch, and the requests behind it in
            // the ring, wait until nothing is in flight (the reference applies the switch at once).
            while (!scheduler_->idle() && !stop_.load(std::memory_order_acquire)) {
                scheduler_->try_handle_block_start_finish();
                job::Context::run_poll_hooks();
            }
            profiler_.handle_cmd();
            break;
        case MsgType::EXIT_CMD: request_stop(); break;
        default: throw std::runtime_error("corrupt request ring: unknown message type " + std::to_string((unsigned)type));
    }
}

void Server::handle_register_client() {
    // The client announces itself under a random temporary id and owns a small reply ring of that name.
    ClientId tmp_id;
    c2s_channel_.read(&tmp_id);
    ipc::ShmChannelCpuWriter reply(ipc::s2c_channel_name(server_name_, tmp_id));

    ClientId id;
    if (unused_client_connections_.empty()) {
        id = (ClientId)client_connections_.size();
        client_connections_.push_back(std::make_unique<ClientConnection>(id));
    } else {
        id = unused_client_connections_.back();
        unused_client_connections_.pop_back();
    }
    ClientConnection* conn = client_connections_[id].get();
    // The permanent completion ring is created here; the client attaches after it learns its id.
    conn->use_s2c_channel(ipc::ShmChannelCpuWriter(ipc::s2c_channel_name(server_name_, id), s2c_channel_size));
    conn->use_s2c_socket(s2c_socket_.connect(ipc::s2c_socket_name(server_name_, id)));
    reply.write(id);
}

void Server::handle_register_job() {
    ClientId client_id;
    c2s_channel_.read(&client_id);
    if (client_id >= client_connections_.size()) throw std::runtime_error("REGISTER_JOB from an unknown client");
    ClientConnection* conn = client_connections_[client_id].get();
    if (unused_registered_jobs_.empty()) {
        const JobRefId id = (JobRefId)registered_jobs_.size();
        registered_jobs_.push_back(std::make_unique<RegisteredJob>(id, &c2s_channel_, conn));
    } else {
        const JobRefId id = unused_registered_jobs_.back();
        unused_registered_jobs_.pop_back();
        registered_jobs_[id]->init(&c2s_channel_, conn);
    }
}

void Server::handle_launch_job() {
    if (ipc::launch_timestamps()) {
        // Mean latency of the request ring (reference src/server/server.cpp:121-141): the first 10 000 requests are left out,
        // then every 1000th prints the running mean.
        unsigned long long sent;
        c2s_channel_.read(&sent);
        if (ipc_latency_skipped_ >= ipc_latency_skip_) {
            const unsigned long long now = (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();
            ipc_latency_sum_ns_ += (double)(now - sent) * (1e9 * (double)std::chrono::steady_clock::period::num / (double)std::chrono::steady_clock::period::den);
            if (++ipc_latency_count_ % 1000 == 0) {
                std::printf("Avg launch job IPC latency: %f us\n", ipc_latency_mean_us());
                std::fflush(stdout);
            }
        } else {
            ++ipc_latency_skipped_;
        }
    }
    JobRefId id;
    c2s_channel_.read(&id);
    if (id >= registered_jobs_.size()) throw std::runtime_error("LAUNCH_JOB for an unknown job type");
    LLIS_PHASE_WARMUP_TICK();
    scheduler_->handle_new_job(registered_jobs_[id]->create_instance());
}

void Server::handle_grow_pool() {
    JobRefId id;
    c2s_channel_.read(&id);
    if (id >= registered_jobs_.size()) throw std::runtime_error("GROW_POOL for an unknown job type");
    registered_jobs_[id]->grow_pool();
}

void Server::notify_job_starts(job::Job* job) {
    // never blocks: a poke that does not fit the client's socket queue is retried from the poll loop
    if (client_connections_[job->get_client_id()]->wake()) ++total_owed_wakeups_;
}

void Server::notify_job_ends(job::Job* job) {
    job->on_complete();
    total_owed_wakeups_ -= client_connections_[job->get_client_id()]->post_completion(job->get_remote_ptr());
}

void Server::release_job_instance(std::unique_ptr<job::Job> job) {
    const JobRefId id = job->get_registered_job_id();
    registered_jobs_[id]->release_instance(std::move(job));
}

void Server::update_job_stage_length(job::Job* job, unsigned stage_id, double len) { registered_jobs_[job->get_registered_job_id()]->update_stage_length(stage_id, len); }
void Server::set_job_stage_resource(job::Job* job, unsigned stage_id, float res) { registered_jobs_[job->get_registered_job_id()]->set_stage_resource(stage_id, res); }
bool Server::has_job_stage_resource(job::Job* job, unsigned stage_id) { return registered_jobs_[job->get_registered_job_id()]->has_stage_resource(stage_id); }
double Server::get_job_remaining_length(job::Job* job, unsigned from_stage) const { return registered_jobs_[job->get_registered_job_id()]->get_remaining_length(from_stage); }
double Server::get_job_remaining_rl(job::Job* job, unsigned from_stage) const { return registered_jobs_[job->get_registered_job_id()]->get_remaining_rl(from_stage); }
const std::vector<double>& Server::get_job_stage_lengths(job::Job* job) const { return registered_jobs_[job->get_registered_job_id()]->get_stage_lengths(); }
const std::vector<float>& Server::get_job_stage_resources(job::Job* job) const { return registered_jobs_[job->get_registered_job_id()]->get_stage_resources(); }

}  // namespace server
}  // namespace llis
