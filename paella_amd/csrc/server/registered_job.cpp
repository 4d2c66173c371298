#include <llis/job/context.h>
#include <llis/server/registered_job.h>
#include <llis/utils/error.h>

#include <dlfcn.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <stdexcept>

namespace llis {
namespace server {

RegisteredJob::RegisteredJob(JobRefId registered_job_id, ipc::ShmChannelCpuReader* c2s_channel, ClientConnection* client_connection)
    : registered_job_id_(registered_job_id) {
    init(c2s_channel, client_connection);
}

void RegisteredJob::init(ipc::ShmChannelCpuReader* c2s_channel, ClientConnection* client_connection) {
    c2s_channel_ = c2s_channel;
    client_connection_ = client_connection;
    s2c_channel_ = client_connection_->get_s2c_channel();

    std::string job_path;
    c2s_channel_->read(&job_path);
    c2s_channel_->read(&shm_name_);

    // RTLD_GLOBAL: the definition and the kernel library it pulls in must share one copy of job::Context.
    void* handle = dlopen(job_path.c_str(), RTLD_LAZY | RTLD_GLOBAL);
    if (!handle) throw std::runtime_error(std::string("cannot load job definition: ") + dlerror());
    init_job_ = reinterpret_cast<InitJobFn>(dlsym(handle, "init_job"));
    if (!init_job_) throw std::runtime_error("job definition " + job_path + " does not export init_job");

    shm_fd_ = shm_open(shm_name_.c_str(), O_RDWR, 0600);
    LLIS_CHECK_POSIX(shm_fd_);

    pool_size_in_bytes_ = 0;
    mapped_mem_.clear();
    unused_job_instances_.clear();
    stage_lengths_.clear();
    stage_resources_.clear();

    s2c_channel_->write(registered_job_id_);
}

std::unique_ptr<job::Job> RegisteredJob::create_instance() {
    int chunk;
    size_t offset;
    void* remote_ptr;
    c2s_channel_->read(&chunk);
    c2s_channel_->read(&offset);
    c2s_channel_->read(&remote_ptr);
    if (chunk < 0 || (size_t)chunk >= mapped_mem_.size()) throw std::runtime_error("LAUNCH_JOB names an unmapped pool chunk");
    void* io_ptr = reinterpret_cast<char*>(mapped_mem_[chunk]) + offset;

    std::unique_ptr<job::Job> job;
    if (unused_job_instances_.empty()) {
        job = init_job();
        job->set_client_details(client_connection_->get_client_id(), registered_job_id_);
        job->set_remote_ptr(remote_ptr);
        job::Context::set_current_job(job.get());
        job->full_init(io_ptr);
    } else {
        job = std::move(unused_job_instances_.back());  // most recently used instance first
        unused_job_instances_.pop_back();
        job->set_remote_ptr(remote_ptr);
        job->reset_internal();
        job::Context::set_current_job(job.get());
        job->init(io_ptr);
    }
    return job;
}

void RegisteredJob::release_instance(std::unique_ptr<job::Job> job) { unused_job_instances_.push_back(std::move(job)); }

void RegisteredJob::grow_pool() {
    size_t num_new_bytes;
    c2s_channel_->read(&num_new_bytes);
    void* p = mmap(nullptr, num_new_bytes, PROT_READ | PROT_WRITE, MAP_SHARED, shm_fd_, (off_t)pool_size_in_bytes_);
    LLIS_CHECK_POSIX_PTR(p, MAP_FAILED);
    // Keep request buffers resident when the limit allows it; jobs stage through runtime-pinned buffers,
    // so a refused mlock costs page faults, not correctness.
    if (mlock(p, num_new_bytes) != 0) {
        static bool warned = false;
        if (!warned) std::fprintf(stderr, "[llis] note: request pool not locked in memory (RLIMIT_MEMLOCK)\n");
        warned = true;
    }
    pool_size_in_bytes_ += num_new_bytes;
    mapped_mem_.push_back(p);
}

std::unique_ptr<job::Job> RegisteredJob::init_job() { return std::unique_ptr<job::Job>(init_job_()); }

void RegisteredJob::update_stage_length(unsigned stage_id, double len) {
    if (stage_id < stage_lengths_.size()) {
        stage_lengths_[stage_id] = (stage_lengths_[stage_id] + len) / 2;
    } else {
        stage_lengths_.push_back(len);
    }
}

void RegisteredJob::set_stage_resource(unsigned stage_id, float res) {
    if (stage_resources_.size() <= stage_id) stage_resources_.push_back(res);
}

bool RegisteredJob::has_stage_resource(unsigned stage_id) { return stage_resources_.size() > stage_id; }

double RegisteredJob::get_stage_length(unsigned stage_id) const { return stage_id < stage_lengths_.size() ? stage_lengths_[stage_id] : 0; }

float RegisteredJob::get_stage_resource(unsigned stage_id) const { return stage_id < stage_resources_.size() ? stage_resources_[stage_id] : 0; }

double RegisteredJob::get_remaining_length(unsigned from_stage) const {
    double sum = 0;
    for (size_t i = from_stage; i < stage_lengths_.size(); ++i) sum += stage_lengths_[i];
    return sum;
}

double RegisteredJob::get_remaining_rl(unsigned from_stage) const {
    double sum = 0;
    for (size_t i = from_stage; i < stage_lengths_.size() && i < stage_resources_.size(); ++i) sum += stage_lengths_[i] * stage_resources_[i];
    return sum;
}

}  // namespace server
}  // namespace llis
