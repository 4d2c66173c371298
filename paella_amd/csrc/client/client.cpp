#include <llis/client/client.h>
#include <llis/ipc/name_format.h>
#include <llis/job/job.h>

#include <dlfcn.h>

#include <random>
#include <stdexcept>

namespace llis {
namespace client {

Client::Client(std::string server_name)
    : server_name_(std::move(server_name)), c2s_channel_(ipc::c2s_channel_name(server_name_)), profiler_client_(&c2s_channel_) {
    // Handshake: announce a random temporary id, own a tiny reply ring under that id, learn the permanent
    // id from it, then attach to the completion ring and bind the wake-up socket the server made for it.
    std::random_device rnd;
    const ClientId tmp_id = rnd();
    s2c_channel_.connect(ipc::s2c_channel_name(server_name_, tmp_id), 8);

    c2s_channel_.acquire_writer_lock();
    c2s_channel_.write(MsgType::REGISTER_CLIENT);
    c2s_channel_.write(tmp_id);
    c2s_channel_.release_writer_lock();

    s2c_channel_.read(&client_id_);
    s2c_channel_.disconnect();
    s2c_channel_.connect(ipc::s2c_channel_name(server_name_, client_id_));
    s2c_socket_.bind(ipc::s2c_socket_name(server_name_, client_id_));
}

Client::~Client() {}

JobRef Client::register_job(std::string path) {
    void* handle = dlopen(path.c_str(), RTLD_NOW);
    if (!handle) throw std::runtime_error(std::string("cannot load job definition: ") + dlerror());
    using InitJobFn = job::Job* (*)();
    InitJobFn init_job = reinterpret_cast<InitJobFn>(dlsym(handle, "init_job"));
    if (!init_job) throw std::runtime_error("job definition " + path + " does not export init_job");
    return JobRef(std::unique_ptr<job::Job>(init_job()), this, path);
}

void Client::send_bare(MsgType type) {
    c2s_channel_.acquire_writer_lock();
    c2s_channel_.write(type);
    c2s_channel_.release_writer_lock();
}

void Client::cuda_profiler_start() { send_bare(MsgType::CUDA_PROFILER_START); }
void Client::cuda_profiler_stop() { send_bare(MsgType::CUDA_PROFILER_STOP); }
void Client::kill_server() { send_bare(MsgType::EXIT_CMD); }

JobInstanceRef* Client::add_job_instance_ref(JobInstanceRef ref) {
    std::lock_guard<std::mutex> lk(mtx_);
    if (unused_job_instance_refs_.empty()) {
        ref.set_id((JobInstanceRefId)job_instance_refs_.size());
        job_instance_refs_.push_back(std::make_unique<JobInstanceRef>(std::move(ref)));
        return job_instance_refs_.back().get();
    }
    const JobInstanceRefId id = unused_job_instance_refs_.back();
    unused_job_instance_refs_.pop_back();
    ref.set_id(id);
    *job_instance_refs_[id] = std::move(ref);
    return job_instance_refs_[id].get();
}

void Client::release_job_instance_ref(JobInstanceRef* ref) {
    std::lock_guard<std::mutex> lk(mtx_);
    unused_job_instance_refs_.push_back(ref->get_id());
}

JobInstanceRef* Client::wait() {
    bool woken;
    s2c_socket_.read(&woken, sizeof(woken));  // sent when the request's last stage is dispatched
    JobInstanceRef* done;
    s2c_channel_.read(&done);  // posted when it has completed
    return done;
}

}  // namespace client
}  // namespace llis
