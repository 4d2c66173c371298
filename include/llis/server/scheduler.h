#pragma once
// Scheduler interface, the name -> factory registry, and the machinery all three policies share: the
// GPU->host notification ring, the copy-completion channel, LIFO pools of streams, notifiers and JobIds.
//
// Policies (reference src/server/CMakeLists.txt builds exactly these three):
//   "fifo"   job by job: all stages of a job are issued at once on one stream          (scheduler_fifo.h)
//   "fifo2"  kernel by kernel in arrival order, no admission control                   (scheduler_fifo2.h)
//   "full3"  kernel by kernel, shortest remaining work first, deficit-counter fairness,
//            occupancy-based admission with bounded over-subscription                  (scheduler_full3.h)
// Interface after reference include/llis/server/scheduler.h:18-45; options replace boost::program_options.

#include <llis/ipc/shm_channel.h>
#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/finished_block_notifier.h>
#include <llis/job/instrument_info.h>
#include <llis/job/job.h>
#include <llis/server/server.h>

#include <functional>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#define GPU2SCHED_CHAN_SIZE 1024000

namespace llis {
namespace server {

struct SchedulerOptions {
    unsigned num_streams = 500;     // --num_streams
    unsigned extra_kernels = 2;     // --extra_kernels: kernels admitted beyond full occupancy (full3)
    float unfair = 1000000.f;       // --unfair: deficit threshold that triggers fairness (full3)
    unsigned sched_sleep = 0;       // --sched_sleep: artificial spin per scheduling decision
    // How a copy stage reports completion: true = a one-lane marker kernel writes into the GPU ring,
    // false = a runtime host callback writes the job pointer into the mem2sched byte ring.
    bool mem_marker = true;
    size_t ring_slots = GPU2SCHED_CHAN_SIZE;
    // --measure_block_time: every workgroup also reports its entry and exit clock through a second ring; the
    // profiler keeps the pairs while block-exec-time recording is on (reference: compile-time LLIS_MEASURE_BLOCK_TIME).
    bool measure_block_time = false;
    // --noti_batch: workgroups covered by one aggregated notification (a power of two, at most 128).  0 = the
    // library's default of 64; 16 is the reference's constant (reference include/llis/job/finished_block_notifier.h:118).
    unsigned noti_batch = 0;
    // --placement per_cu (full3): admission asks the per-compute-unit model (GpuResources: does every XCD have room for
    // its share of the grid) instead of the pooled budget, predicts where the workgroups will land and, for kernels that
    // report through the un-aggregated hooks, reconciles the prediction with the compute unit each message names.
    bool per_cu_placement = false;
};

class Scheduler {
  public:
    virtual ~Scheduler() {}
    virtual void set_server(Server* server) {
        server_ = server;
        profiler_ = server->get_profiler();
        log_ = server->get_event_log();
    }
    virtual void try_handle_block_start_finish() = 0;
    virtual void handle_new_job(std::unique_ptr<job::Job> job) = 0;
    // No job is in flight: every job handed over has had its last stage's completion handled.
    virtual bool idle() const { return true; }

  protected:
    Server* server_ = nullptr;
    Profiler* profiler_ = nullptr;
    EventLog* log_ = nullptr;
};

class SchedulerFactory {
  public:
    using RegisterFunc = std::function<std::unique_ptr<Scheduler>(const SchedulerOptions&)>;
    static bool register_scheduler(std::string name, RegisterFunc func);
    // Throws std::invalid_argument for an unknown name.
    static std::unique_ptr<Scheduler> create(std::string name, const SchedulerOptions& options);
    static std::vector<std::string> names();

  private:
    static std::unordered_map<std::string, RegisterFunc>& registry();
};

#define LLIS_SCHEDULER_REGISTER(name, func) \
    static bool __scheduler_register_ = ::llis::server::SchedulerFactory::register_scheduler(name, func);

// Shared plumbing of the stream-pool schedulers.
class StreamPoolScheduler : public Scheduler {
  public:
    void try_handle_block_start_finish() final;
    bool idle() const final { return num_jobs_ == 0; }

  protected:
    StreamPoolScheduler(const SchedulerOptions& options, size_t mem2sched_bytes);
    ~StreamPoolScheduler() override;

    virtual void handle_block_start(job::Job* job, unsigned num) = 0;
    virtual void handle_block_finish(job::Job* job, unsigned num) = 0;
    virtual void handle_mem_finish(job::Job* job) = 0;

    // Gives the job a JobId (most recently freed first) and takes ownership.
    job::Job* adopt(std::unique_ptr<job::Job> job);
    // Frees the JobId and hands the instance back to its RegisteredJob pool.
    void retire(job::Job* job);
    job::Job* job_of(JobId id) { return job_id_to_job_map_[id].get(); }

    bool has_stream() const { return !free_streams_.empty(); }
    // LIFO: the stream / notifier returned last is handed out first.
    unsigned take_stream() { unsigned s = free_streams_.back(); free_streams_.pop_back(); return s; }
    void give_stream(job::Job* job);
    unsigned take_notifier() { unsigned n = free_notifiers_.back(); free_notifiers_.pop_back(); return n; }
    void give_notifier(job::Job* job);
    job::StreamHandle stream_handle(unsigned idx) const { return reinterpret_cast<job::StreamHandle>(streams_[idx]); }
    job::FinishedBlockNotifier* notifier_ptr(unsigned idx) const { return notifiers_raw_ + idx; }

    // Arranges for handle_mem_finish(job) once everything issued so far on the job's stream has completed.
    void post_mem_completion(job::Job* job);
    void spin_sleep() const;

    SchedulerOptions options_;
    unsigned num_jobs_ = 0;
    // Compute-unit id of the message being handled (InstrumentInfo.smid): meaningful inside handle_block_start / _finish for
    // stages whose kernels use the un-aggregated hooks.
    unsigned cur_smid_ = 0;

  private:
    static void mem_notification_callback(void* job);

    ipc::Gpu2SchedChannel gpu2sched_channel_;
    ipc::Gpu2SchedChannel gpu2sched_block_time_channel_;  // connected only with options.measure_block_time
    ipc::ShmChannelCpuReader mem2sched_channel_;
    std::vector<void*> streams_;
    std::vector<unsigned> free_streams_;
    job::FinishedBlockNotifier* notifiers_raw_ = nullptr;
    std::vector<unsigned> free_notifiers_;
    std::unordered_map<void*, unsigned> stream_index_;
    std::vector<std::unique_ptr<job::Job>> job_id_to_job_map_;
    std::vector<JobId> unused_job_id_;
};

}  // namespace server
}  // namespace llis
