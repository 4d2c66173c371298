#pragma once
// Client-side handle of one reusable request slot of a registered job type: fill get_input_ptr(), call
// launch(), and after Client::wait() returns this handle read get_output_ptr()
// (reference include/llis/client/job_instance_ref.h, src/client/job_instance_ref.cpp:14-69).

#include <llis/client/io_shm_entry.h>
#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>

namespace llis {
namespace client {

class JobRef;

class JobInstanceRef {
  public:
    JobInstanceRef(JobRef* job_ref, IoShmEntry io_shm_entry);
    ~JobInstanceRef() {}

    // Sends LAUNCH_JOB{job type, pool chunk, offset, this}; `this` comes back through Client::wait().
    void launch();
    // Returns the slot to the job type's free list.
    void release();

    void* get_input_ptr();
    // The output starts right after the input bytes (not at the 8-byte-aligned offset).
    void* get_output_ptr();

    void set_id(JobInstanceRefId id) { id_ = id; }
    JobInstanceRefId get_id() const { return id_; }
    JobRefId get_job_ref_id() const;

    // Free-form timestamp kept for the caller's latency arithmetic.
    void set_start_time(double time_point) { start_time_ = time_point; }
    double get_start_time() const { return start_time_; }

  private:
    JobRef* job_ref_;
    IoShmEntry io_shm_entry_;
    JobInstanceRefId id_ = 0;
    ipc::ShmChannelCpuWriter* c2s_channel_;
    double start_time_ = 0;
};

}  // namespace client
}  // namespace llis
