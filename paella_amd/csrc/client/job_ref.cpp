#include <llis/client/client.h>
#include <llis/client/job_ref.h>
#include <llis/utils/error.h>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cstdint>
#include <stdexcept>

namespace llis {
namespace client {

JobRef::JobRef(std::unique_ptr<job::Job> job, Client* client, std::string path) : job_(std::move(job)), client_(client), model_path_(std::move(path)) {
    pinned_mem_size_ = job_->get_pinned_mem_size();
    if (pinned_mem_size_ == 0 || pinned_mem_size_ > kPoolChunkBytes) throw std::invalid_argument("request slot does not fit a pool chunk");
    s2c_channel_ = client_->get_s2c_channel();
    c2s_channel_ = client_->get_c2s_channel();
    client_id_ = client_->get_client_id();

    // The name has to be unique among the live pools of this client.  The reference takes the address of this object
    // (reference src/client/job_ref.cpp:24), but register_job() returns by value: two calls from one loop build their objects in
    // the same stack slot, get the same name, and both job types' request slots then alias one shared-memory object (every
    // answer of one type can be overwritten by the other's inputs).  A per-process counter under the process id cannot repeat.
    static std::atomic<uint64_t> next_pool{0};
    shm_name_ = "llis:shm:" + std::to_string(client_id_) + ":" + std::to_string(((uint64_t)getpid() << 24) + next_pool.fetch_add(1));
    shm_unlink(shm_name_.c_str());  // a leftover of a killed process that had this pid
    shm_fd_ = shm_open(shm_name_.c_str(), O_CREAT | O_EXCL | O_RDWR, 0600);
    LLIS_CHECK_POSIX(shm_fd_);

    register_job();
    grow_pool();
}

JobRef::~JobRef() { close_pool(); }

void JobRef::close_pool() {
    if (shm_fd_ == -1) return;  // moved-from
    for (void* p : pinned_mem_list_) munmap(p, kPoolChunkBytes);
    pinned_mem_list_.clear();
    close(shm_fd_);
    shm_unlink(shm_name_.c_str());
    shm_fd_ = -1;
}

void JobRef::steal(JobRef& rhs) {
    job_ = std::move(rhs.job_);
    client_ = rhs.client_;
    model_path_ = std::move(rhs.model_path_);
    s2c_channel_ = rhs.s2c_channel_;
    c2s_channel_ = rhs.c2s_channel_;
    client_id_ = rhs.client_id_;
    pinned_mem_size_ = rhs.pinned_mem_size_;
    pool_size_in_bytes_ = rhs.pool_size_in_bytes_;
    pinned_mem_list_ = std::move(rhs.pinned_mem_list_);
    pinned_mem_free_list_ = std::move(rhs.pinned_mem_free_list_);
    shm_name_ = std::move(rhs.shm_name_);
    shm_fd_ = rhs.shm_fd_;
    job_ref_id_ = rhs.job_ref_id_;
    rhs.shm_fd_ = -1;
    rhs.pinned_mem_list_.clear();
}

void JobRef::register_job() {
    c2s_channel_->acquire_writer_lock();
    c2s_channel_->write(MsgType::REGISTER_JOB);
    c2s_channel_->write(client_id_);
    c2s_channel_->write(model_path_);
    c2s_channel_->write(shm_name_);
    c2s_channel_->release_writer_lock();
    s2c_channel_->read(&job_ref_id_);
}

JobInstanceRef* JobRef::create_instance() {
    if (pinned_mem_free_list_.empty()) grow_pool();
    JobInstanceRef ref(this, pinned_mem_free_list_.back());
    pinned_mem_free_list_.pop_back();
    return client_->add_job_instance_ref(std::move(ref));
}

void JobRef::release_io_shm_entry(IoShmEntry entry) { pinned_mem_free_list_.push_back(entry); }

void JobRef::grow_pool() {
    const size_t old_bytes = pool_size_in_bytes_;
    pool_size_in_bytes_ += kPoolChunkBytes;
    LLIS_CHECK_POSIX(ftruncate(shm_fd_, (off_t)pool_size_in_bytes_));
    void* chunk = mmap(nullptr, kPoolChunkBytes, PROT_READ | PROT_WRITE, MAP_SHARED, shm_fd_, (off_t)old_bytes);
    LLIS_CHECK_POSIX_PTR(chunk, MAP_FAILED);
    pinned_mem_list_.push_back(chunk);

    const int chunk_id = (int)pinned_mem_list_.size() - 1;
    const size_t slots = kPoolChunkBytes / pinned_mem_size_;
    for (size_t i = 0; i < slots; ++i) {
        const size_t offset = i * pinned_mem_size_;
        pinned_mem_free_list_.push_back(IoShmEntry{reinterpret_cast<char*>(chunk) + offset, chunk_id, offset});
    }

    c2s_channel_->acquire_writer_lock();
    c2s_channel_->write(MsgType::GROW_POOL);
    c2s_channel_->write(job_ref_id_);
    c2s_channel_->write(kPoolChunkBytes);
    c2s_channel_->release_writer_lock();
}

}  // namespace client
}  // namespace llis
