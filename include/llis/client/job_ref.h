#pragma once
// A job type registered with the server, and the client's side of its request pool: a POSIX shared
// memory object "llis:shm:<client id>:<address>" grown in chunks that the server maps too, carved into
// fixed-size slots of align8(input) + align8(output) bytes
// (reference include/llis/client/job_ref.h, src/client/job_ref.cpp:16-105).

#include <llis/client/job_instance_ref.h>
#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/job/job.h>

#include <memory>
#include <string>
#include <vector>

namespace llis {
namespace client {

class Client;

class JobRef {
  public:
    // Size of every pool chunk in bytes (a constant, whatever the slot size, like the reference's).
    static constexpr size_t kPoolChunkBytes = 30638080;

    JobRef(std::unique_ptr<job::Job> job, Client* client, std::string path);
    ~JobRef();

    JobRef(const JobRef&) = delete;
    JobRef& operator=(const JobRef&) = delete;
    JobRef(JobRef&& rhs) { steal(rhs); }
    JobRef& operator=(JobRef&& rhs) {
        if (this != &rhs) {
            close_pool();
            steal(rhs);
        }
        return *this;
    }

    JobInstanceRef* create_instance();
    void release_io_shm_entry(IoShmEntry io_shm_entry);

    job::Job* get_job() { return job_.get(); }
    Client* get_client() { return client_; }
    ClientId get_client_id() const { return client_id_; }
    JobRefId get_job_ref_id() const { return job_ref_id_; }
    ipc::ShmChannelCpuReader* get_s2c_channel() { return s2c_channel_; }
    ipc::ShmChannelCpuWriter* get_c2s_channel() { return c2s_channel_; }

  private:
    void register_job();
    void grow_pool();
    void close_pool();
    void steal(JobRef& rhs);

    std::unique_ptr<job::Job> job_;   // local instance, only asked for its sizes
    Client* client_;
    std::string model_path_;

    ipc::ShmChannelCpuReader* s2c_channel_;
    ipc::ShmChannelCpuWriter* c2s_channel_;
    ClientId client_id_;

    size_t pinned_mem_size_;
    size_t pool_size_in_bytes_ = 0;
    std::vector<void*> pinned_mem_list_;
    std::vector<IoShmEntry> pinned_mem_free_list_;

    std::string shm_name_;
    int shm_fd_ = -1;
    JobRefId job_ref_id_ = 0;
};

}  // namespace client
}  // namespace llis
