#pragma once
// The serving process: one busy-polling thread that alternates between the client request ring and the
// scheduler's completion channels (reference include/llis/server/server.h, src/server/server.cpp:24-199).

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>
#include <llis/server/client_connection.h>
#include <llis/server/event_log.h>
#include <llis/server/profiler.h>
#include <llis/server/registered_job.h>

#include <atomic>
#include <memory>
#include <string>
#include <vector>

namespace llis {
namespace server {

class Scheduler;

constexpr size_t c2s_channel_size = 1024;
constexpr size_t s2c_channel_size = 4096;

class Server {
  public:
    Server(std::string server_name, Scheduler* scheduler);
    ~Server();

    // Polls until an EXIT_CMD arrives or request_stop() is called.
    void serve();
    // One iteration of the poll loop (request ring, then completion channels).
    void poll_once();
    void request_stop() { stop_.store(true, std::memory_order_release); }

    void notify_job_starts(job::Job* job);
    void notify_job_ends(job::Job* job);
    void release_job_instance(std::unique_ptr<job::Job> job);

    void update_job_stage_length(job::Job* job, unsigned stage_id, double len);
    void set_job_stage_resource(job::Job* job, unsigned stage_id, float res);
    bool has_job_stage_resource(job::Job* job, unsigned stage_id);
    double get_job_remaining_length(job::Job* job, unsigned from_stage) const;
    double get_job_remaining_rl(job::Job* job, unsigned from_stage) const;
    const std::vector<double>& get_job_stage_lengths(job::Job* job) const;
    const std::vector<float>& get_job_stage_resources(job::Job* job) const;

    Profiler* get_profiler() { return &profiler_; }
    EventLog* get_event_log() { return &event_log_; }
    const std::string& get_name() const { return server_name_; }
    // With ipc::launch_timestamps(): mean client-to-server latency of LAUNCH_JOB in microseconds and how many requests it covers.
    double ipc_latency_mean_us() const { return ipc_latency_count_ ? ipc_latency_sum_ns_ / (double)ipc_latency_count_ / 1e3 : 0.0; }
    uint64_t ipc_latency_count() const { return ipc_latency_count_; }

  private:
    void handle_c2s();
    void handle_register_client();
    void handle_register_job();
    void handle_launch_job();
    void handle_grow_pool();
    void retry_owed_wakeups();

    std::string server_name_;
    Scheduler* scheduler_;
    ipc::UnixDatagramSocket s2c_socket_;
    ipc::ShmChannelCpuReader c2s_channel_;

    // unique_ptr: RegisteredJob keeps pointers to its ClientConnection across growth of these vectors.
    std::vector<std::unique_ptr<ClientConnection>> client_connections_;
    std::vector<ClientId> unused_client_connections_;
    std::vector<std::unique_ptr<RegisteredJob>> registered_jobs_;
    std::vector<JobRefId> unused_registered_jobs_;

    Profiler profiler_;
    EventLog event_log_;
    std::atomic<bool> stop_{false};
    unsigned total_owed_wakeups_ = 0;
    unsigned polls_since_retry_ = 0;

    unsigned ipc_latency_skip_ = 10000, ipc_latency_skipped_ = 0;  // LLIS_IPC_LATENCY_SKIP overrides the reference's 10 000
    uint64_t ipc_latency_count_ = 0;
    double ipc_latency_sum_ns_ = 0;
};

}  // namespace server
}  // namespace llis
