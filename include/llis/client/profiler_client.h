#pragma once
// Client-side switches of the server's recorder (reference include/llis/client/profiler_client.h,
// src/client/profiler_client.cpp:7-123): each call sends PROFILER_CMD + a sub-command on the request ring.

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>

#include <string>

namespace llis {
namespace client {

class ProfilerClient {
  public:
    explicit ProfilerClient(ipc::ShmChannelCpuWriter* c2s_channel) : c2s_channel_(c2s_channel) {}

    void set_record_kernel_info() { send(ProfilerMsgType::SET_RECORD_KERNEL_INFO); }
    void unset_record_kernel_info() { send(ProfilerMsgType::UNSET_RECORD_KERNEL_INFO); }
    void set_record_block_exec_time() { send(ProfilerMsgType::SET_RECORD_BLOCK_EXEC_TIME); }
    void unset_record_block_exec_time() { send(ProfilerMsgType::UNSET_RECORD_BLOCK_EXEC_TIME); }
    void set_record_kernel_block_mis_alloc() { send(ProfilerMsgType::SET_RECORD_KERNEL_BLOCK_MIS_ALLOC); }
    void unset_record_kernel_block_mis_alloc() { send(ProfilerMsgType::UNSET_RECORD_KERNEL_BLOCK_MIS_ALLOC); }
    void set_record_run_next_times() { send(ProfilerMsgType::SET_RECORD_RUN_NEXT_TIMES); }
    void unset_record_run_next_times() { send(ProfilerMsgType::UNSET_RECORD_RUN_NEXT_TIMES); }
    void set_record_job_events() { send(ProfilerMsgType::SET_RECORD_JOB_EVENTS); }
    void unset_record_job_events() { send(ProfilerMsgType::UNSET_RECORD_JOB_EVENTS); }
    void set_record_resource_events() { send(ProfilerMsgType::SET_RECORD_RESOURCE_EVENTS); }
    void unset_record_resource_events() { send(ProfilerMsgType::UNSET_RECORD_RESOURCE_EVENTS); }

    // Asks the server to write its recordings to files starting with `path`.
    void save(const std::string& path);

  private:
    void send(ProfilerMsgType sub);
    ipc::ShmChannelCpuWriter* c2s_channel_;
};

}  // namespace client
}  // namespace llis
