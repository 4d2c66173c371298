#pragma once
// One job type registered by a client: the loaded job definition (dlopen + init_job), the client's
// shared-memory request pool mapped into the server, a LIFO pool of reusable job instances, and the
// learned per-stage lengths that drive shortest-remaining-work priorities
// (reference include/llis/server/registered_job.h, src/server/registered_job.cpp:20-184).

#include <llis/ipc/shm_channel.h>
#include <llis/job/job.h>
#include <llis/server/client_connection.h>

#include <memory>
#include <string>
#include <vector>

namespace llis {
namespace server {

class RegisteredJob {
  public:
    using InitJobFn = job::Job* (*)();

    // Reads {job path, pool shm name} from the request ring, loads the definition and answers with the id.
    RegisteredJob(JobRefId registered_job_id, ipc::ShmChannelCpuReader* c2s_channel, ClientConnection* client_connection);
    RegisteredJob(RegisteredJob&&) = default;
    RegisteredJob& operator=(RegisteredJob&&) = default;

    void init(ipc::ShmChannelCpuReader* c2s_channel, ClientConnection* client_connection);

    // Reads {pool chunk id, offset, client cookie} of a LAUNCH_JOB and returns a ready instance whose
    // first stage has been declared.
    std::unique_ptr<job::Job> create_instance();
    // Reads the size of a GROW_POOL and maps the new chunk of the client's pool.
    void grow_pool();
    std::unique_ptr<job::Job> init_job();
    void release_instance(std::unique_ptr<job::Job> job);

    // Running estimate of stage `stage_id`'s length in microseconds: first sample, then (old + new) / 2.
    void update_stage_length(unsigned stage_id, double len);
    void set_stage_resource(unsigned stage_id, float res);
    bool has_stage_resource(unsigned stage_id);
    double get_stage_length(unsigned stage_id) const;   // 0 while unknown
    float get_stage_resource(unsigned stage_id) const;  // 0 while unknown
    double get_remaining_length(unsigned from_stage) const;
    double get_remaining_rl(unsigned from_stage) const;  // sum of length x resource over learned stages

    const std::vector<double>& get_stage_lengths() const { return stage_lengths_; }
    const std::vector<float>& get_stage_resources() const { return stage_resources_; }

  private:
    JobRefId registered_job_id_;
    ipc::ShmChannelCpuReader* c2s_channel_ = nullptr;
    ClientConnection* client_connection_ = nullptr;
    ipc::ShmChannelCpuWriter* s2c_channel_ = nullptr;

    InitJobFn init_job_ = nullptr;
    std::string shm_name_;
    int shm_fd_ = -1;
    size_t pool_size_in_bytes_ = 0;
    std::vector<void*> mapped_mem_;

    std::vector<std::unique_ptr<job::Job>> unused_job_instances_;
    std::vector<double> stage_lengths_;
    std::vector<float> stage_resources_;
};

}  // namespace server
}  // namespace llis
