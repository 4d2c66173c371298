#include <llis/client/job_instance_ref.h>
#include <llis/client/job_ref.h>
#include <llis/ipc/defs.h>

#include <chrono>

namespace llis {
namespace client {

namespace {

// LAUNCH_JOB as it travels on the request ring (reference src/client/job_instance_ref.cpp:31-45 writes the same five
// values one after the other; the ring is a byte stream, so one packed record is the same bytes under one lock).
#pragma pack(push, 1)
struct LaunchRecord {
    MsgType type;
    JobRefId job_ref_id;
    int pool_id;
    size_t offset;
    JobInstanceRef* handle;   // comes back on the completion ring when the request is done
};
#pragma pack(pop)
static_assert(sizeof(LaunchRecord) == 4 + 4 + 4 + 8 + 8, "LAUNCH_JOB is 28 bytes on the wire");

// The same with the send time behind the type (reference src/client/job_instance_ref.cpp:35-38 under
// PRINT_LAUNCH_JOB_IPC_LATENCY): steady_clock ticks since its epoch, which every process of the machine shares.
#pragma pack(push, 1)
struct TimedLaunchRecord {
    MsgType type;
    unsigned long long send_time;
    JobRefId job_ref_id;
    int pool_id;
    size_t offset;
    JobInstanceRef* handle;
};
#pragma pack(pop)
static_assert(sizeof(TimedLaunchRecord) == 4 + 8 + 4 + 4 + 8 + 8, "LAUNCH_JOB with a send time is 36 bytes on the wire");

}  // namespace

JobInstanceRef::JobInstanceRef(JobRef* job_ref, IoShmEntry io_shm_entry) : job_ref_(job_ref), io_shm_entry_(io_shm_entry) {
    c2s_channel_ = job_ref_->get_c2s_channel();
}

void* JobInstanceRef::get_input_ptr() { return io_shm_entry_.ptr; }

// The output follows the input in the request slot.
void* JobInstanceRef::get_output_ptr() { return static_cast<char*>(get_input_ptr()) + job_ref_->get_job()->get_input_size(); }

void JobInstanceRef::launch() {
    if (ipc::launch_timestamps()) {
        TimedLaunchRecord rec;
        rec.type = MsgType::LAUNCH_JOB;
        rec.job_ref_id = job_ref_->get_job_ref_id();
        rec.pool_id = io_shm_entry_.id;
        rec.offset = io_shm_entry_.offset;
        rec.handle = this;
        c2s_channel_->acquire_writer_lock();
        rec.send_time = (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();  // under the lock, like the reference
        c2s_channel_->write(&rec, sizeof(rec));
        c2s_channel_->release_writer_lock();
        return;
    }
    LaunchRecord rec;
    rec.type = MsgType::LAUNCH_JOB;
    rec.job_ref_id = job_ref_->get_job_ref_id();
    rec.pool_id = io_shm_entry_.id;
    rec.offset = io_shm_entry_.offset;
    rec.handle = this;
    c2s_channel_->acquire_writer_lock();
    c2s_channel_->write(&rec, sizeof(rec));
    c2s_channel_->release_writer_lock();
}

void JobInstanceRef::release() { job_ref_->release_io_shm_entry(io_shm_entry_); }

JobRefId JobInstanceRef::get_job_ref_id() const { return job_ref_->get_job_ref_id(); }

}  // namespace client
}  // namespace llis
