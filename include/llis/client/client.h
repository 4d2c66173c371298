#pragma once
// llis::client::Client -- connection of an application process to a named server
// (reference include/llis/client/client.h:16-47, src/client/client.cpp:19-136).
//
//   Client client("srv");
//   JobRef job = client.register_job("/path/libjob_x.so");
//   JobInstanceRef* inst = job.create_instance();
//   fill(inst->get_input_ptr());  inst->launch();
//   JobInstanceRef* done = client.wait();   // blocks; returns the instance that finished
//
// launch() may be called from one thread while another blocks in wait().

#include <llis/client/job_ref.h>
#include <llis/client/profiler_client.h>
#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>

#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace llis {
namespace client {

class Client {
  public:
    explicit Client(std::string server_name);
    ~Client();

    // Loads the job definition locally (for its sizes) and registers it with the server.
    JobRef register_job(std::string path);

    ClientId get_client_id() const { return client_id_; }
    ipc::ShmChannelCpuWriter* get_c2s_channel() { return &c2s_channel_; }
    ipc::ShmChannelCpuReader* get_s2c_channel() { return &s2c_channel_; }

    void cuda_profiler_start();
    void cuda_profiler_stop();

    JobInstanceRef* add_job_instance_ref(JobInstanceRef job_instance_ref);
    void release_job_instance_ref(JobInstanceRef* job_instance_ref);

    // Sleeps on the wake-up socket, then spins on the completion ring for the finished instance.
    JobInstanceRef* wait();

    ProfilerClient* get_profiler_client() { return &profiler_client_; }

    void kill_server();

  private:
    void send_bare(MsgType type);

    std::string server_name_;
    ClientId client_id_ = 0;
    ipc::ShmChannelCpuWriter c2s_channel_;
    ipc::ShmChannelCpuReader s2c_channel_;
    ipc::UnixDatagramSocket s2c_socket_;

    std::vector<std::unique_ptr<JobInstanceRef>> job_instance_refs_;
    std::vector<JobInstanceRefId> unused_job_instance_refs_;
    std::mutex mtx_;

    ProfilerClient profiler_client_;
};

}  // namespace client
}  // namespace llis
