#pragma once
// llis::job::Job -- one in-flight request, as seen by the scheduler.
//
// A job is a sequence of stages.  Before the scheduler resumes it for stage i (run_next()), the job has
// already DECLARED what stage i needs: whether it is a copy stage (is_mem) or a kernel, and for a kernel
// its grid size, workgroup size, LDS per workgroup and registers per thread.  When resumed it issues
// exactly one asynchronous GPU operation on get_cuda_stream(), passing get_id() and
// get_finished_block_notifier() to the kernel, then declares the next stage and returns.
//
// The public member names and their meaning follow reference include/llis/job/job.h:16-336 so that job
// definitions written against the reference compile unchanged.  `cudaStream_t` is kept as the spelling
// of the opaque stream handle; on this platform it is a hipStream_t.

#include <llis/ipc/defs.h>
#include <llis/job/finished_block_notifier.h>
#include <llis/utils/align.h>

#include <chrono>
#include <cstddef>
#include <vector>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
namespace llis { namespace job { using StreamHandle = hipStream_t; } }
#else
namespace llis { namespace job { using StreamHandle = void*; } }
#endif

#ifndef LLIS_NO_CUDA_SPELLINGS
// Job definitions written for the reference name the stream type this way.
using cudaStream_t = llis::job::StreamHandle;
#endif

namespace llis {
namespace job {

// What one stage asks of the GPU.
struct StageNeeds {
    unsigned num_blocks = 0;
    unsigned num_threads_per_block = 0;
    unsigned smem_size_per_block = 0;
    unsigned num_registers_per_thread = 0;
};

class Job {
  public:
    using Clock = std::chrono::steady_clock;

    virtual ~Job() {}

    // ---- implemented by the job definition
    virtual size_t get_input_size() = 0;
    virtual size_t get_output_size() = 0;
    virtual size_t get_param_size() = 0;
    virtual void full_init(void* io_ptr) = 0;  // first use of a pooled instance
    virtual void init(void* io_ptr) = 0;       // every later reuse
    virtual void run_next() = 0;
    virtual bool has_next() const = 0;
    // Called by the server on its own thread after the last stage has completed and before the client is
    // told.  Default: nothing.  (Extension: request buffers of the client pool cannot be made
    // device-visible on every platform, so a job may need to copy results out of a staging buffer.)
    virtual void on_complete() {}

    // ---- bookkeeping used by the server; a recycled instance starts from here
    void reset_internal() {
        is_running_ = false;
        has_started_ = false;
        is_mem_ = false;
        is_pre_notify_ = false;
        completes_itself_ = false;
        is_unfit_ = false;
        deficit_counter_ = 0;
        cur_stage_ = -1;
    }

    void set_id(JobId id) {
        static unsigned next_unique_id = 0;
        id_ = id;
        unique_id_ = next_unique_id++;  // arrival order across all jobs of the process
    }
    JobId get_id() const { return id_; }
    JobId get_unique_id() const { return unique_id_; }
    int get_cur_stage() const { return cur_stage_; }

    // Request slot layout in the client's shared-memory pool: input, then output at the next 8-byte boundary.
    size_t get_output_offset() { return utils::next_aligned_pos(get_input_size(), 8); }
    size_t get_pinned_mem_size() { return get_output_offset() + utils::next_aligned_pos(get_output_size(), 8); }

    // ---- declaration of the NEXT stage
    unsigned get_num_blocks() const { return next_.num_blocks; }
    unsigned get_num_threads_per_block() const { return next_.num_threads_per_block; }
    unsigned get_smem_size_per_block() const { return next_.smem_size_per_block; }
    unsigned get_num_registers_per_thread() const { return next_.num_registers_per_thread; }
    void set_num_blocks(unsigned v) { next_.num_blocks = v; }
    void set_num_threads_per_block(unsigned v) { next_.num_threads_per_block = v; }
    void set_smem_size_per_block(unsigned v) { next_.smem_size_per_block = v; }
    void set_num_registers_per_thread(unsigned v) { next_.num_registers_per_thread = v; }

    bool is_mem() const { return is_mem_; }
    void set_is_mem() { is_mem_ = true; }
    void unset_is_mem() { is_mem_ = false; }

    bool is_pre_notify() const { return is_pre_notify_; }
    void set_pre_notify() { is_pre_notify_ = true; }
    void unset_pre_notify() { is_pre_notify_ = false; }

    // A copy stage that reports its own completion: the job does the stage's work off the serving thread (a host-side copy
    // handed to a helper thread, say) and calls Context::post_mem_completion(this) when it is done, from any thread; the
    // scheduler then posts no completion marker behind the stage.  Only under a scheduler that issues stage by stage
    // (Context::is_stage_by_stage()).  Not in the reference, whose copy stages are all stream operations.
    bool completes_itself() const { return completes_itself_; }
    void set_completes_itself() { completes_itself_ = true; }
    void unset_completes_itself() { completes_itself_ = false; }

    // ---- snapshot of the stage that is currently on the GPU
    unsigned get_cur_num_blocks() const { return cur_.num_blocks; }
    unsigned get_cur_num_threads_per_block() const { return cur_.num_threads_per_block; }
    unsigned get_cur_smem_size_per_block() const { return cur_.smem_size_per_block; }
    unsigned get_cur_num_registers_per_thread() const { return cur_.num_registers_per_thread; }

    bool is_running() const { return is_running_; }
    void unset_running() { is_running_ = false; }

    // The scheduler is about to resume the job for its next stage on `stream`.
    void set_running(StreamHandle stream) {
        is_running_ = true;
        cuda_stream_ = stream;
        cur_ = next_;
        num_running_blocks_ = next_.num_blocks;
        num_pending_blocks_ = next_.num_blocks;
        clear_predicted_smids();
        stage_start_time_ = Clock::now();
        ++cur_stage_;
    }

    StreamHandle get_cuda_stream() const { return cuda_stream_; }

    void set_finished_block_notifier(FinishedBlockNotifier* notifier) {
        finished_block_notifier_ = notifier;
        notifier_read_ = false;
    }
    FinishedBlockNotifier* get_finished_block_notifier() {
        notifier_read_ = true;
        return finished_block_notifier_;
    }
    // False after run_next() if the stage did not ask for its notifier: its kernel then reports through the un-aggregated hooks
    // (llis/job/instrument.h), one message per workgroup that names the compute unit it ran on.  A scheduler that places
    // workgroups per compute unit records that with set_reports_cu() and reads reports_cu() when the messages come in.
    bool used_finished_block_notifier() const { return notifier_read_; }
    bool reports_cu() const { return reports_cu_; }
    void set_reports_cu(bool v) { reports_cu_ = v; }

    Clock::time_point get_stage_start_time() const { return stage_start_time_; }

    // A start message covering `num` workgroups arrived; true while some are still not resident.
    bool mark_block_start() { return mark_block_start(1); }
    bool mark_block_start(unsigned num) {
        num_pending_blocks_ -= num;
        return num_pending_blocks_ != 0;
    }

    // An end message covering `num` workgroups arrived; the stage is over when none remain.
    void mark_block_finish() { mark_block_finish(1); }
    void mark_block_finish(unsigned num) {
        num_running_blocks_ -= num;
        if (num_running_blocks_ == 0) is_running_ = false;
    }

    bool has_started() const { return has_started_; }
    void set_started() { has_started_ = true; }
    void unset_started() { has_started_ = false; }

    void set_client_details(ClientId client_id, JobRefId registered_job_id) {
        client_id_ = client_id;
        registered_job_id_ = registered_job_id;
    }
    ClientId get_client_id() const { return client_id_; }
    JobRefId get_registered_job_id() const { return registered_job_id_; }

    void* get_remote_ptr() const { return remote_ptr_; }
    void set_remote_ptr(void* p) { remote_ptr_ = p; }

    // Per-compute-unit placement prediction of the running stage (reference include/llis/job/job.h:179-199), sized for the 8-bit cu id.
    static constexpr unsigned kMaxCuIds = 256;
    void add_predicted_smid(unsigned smid) {
        ++predicted_smid_nums_[smid % kMaxCuIds];
        any_predicted_ = true;
    }
    const unsigned* get_predicted_smid_nums() const { return predicted_smid_nums_; }
    bool has_predicted_smid(unsigned smid) const { return predicted_smid_nums_[smid % kMaxCuIds] > 0; }
    void dec_predicted_smid(unsigned smid) { --predicted_smid_nums_[smid % kMaxCuIds]; }
    void clear_predicted_smids() {
        if (!any_predicted_) return;
        for (unsigned& n : predicted_smid_nums_) n = 0;
        any_predicted_ = false;
    }

    void inc_deficit_counter(float v) { deficit_counter_ += v; }
    float get_deficit_counter() const { return deficit_counter_; }

    void set_priority(double p) { priority_ = p; }
    double get_priority() const { return priority_; }

    bool is_unfit() const { return is_unfit_; }
    void set_unfit() { is_unfit_ = true; }
    void unset_unfit() { is_unfit_ = false; }

    // Shortest-remaining-work bookkeeping: `total` is the learned sum of length*resource over all stages.
    void set_stage_lengths_resources(double total, const std::vector<double>& lengths, const std::vector<float>& resources) {
        cur_rl_ = total;
        stage_lengths_ = lengths;
        stage_resources_ = resources;
    }
    double get_cur_rl() const { return cur_rl_; }
    // Removes the stage that is about to be queued (cur_stage + 1) from the remaining work.
    void dec_cur_rl() {
        // A stage whose length has not been learned yet counts as zero work.
        const size_t next = (size_t)(cur_stage_ + 1);
        if (next < stage_lengths_.size() && next < stage_resources_.size()) cur_rl_ -= stage_lengths_[next] * stage_resources_[next];
    }

  private:
    StageNeeds next_;
    StageNeeds cur_;
    bool is_mem_ = false;
    bool is_pre_notify_ = false;
    bool completes_itself_ = false;
    bool is_running_ = false;
    bool has_started_ = false;
    bool is_unfit_ = false;
    bool any_predicted_ = true;
    bool notifier_read_ = false;
    bool reports_cu_ = false;

    StreamHandle cuda_stream_ = nullptr;
    FinishedBlockNotifier* finished_block_notifier_ = nullptr;

    unsigned num_running_blocks_ = 0;
    unsigned num_pending_blocks_ = 0;
    unsigned predicted_smid_nums_[kMaxCuIds] = {};

    float deficit_counter_ = 0;
    double priority_ = 0;
    int cur_stage_ = -1;

    std::vector<double> stage_lengths_;
    std::vector<float> stage_resources_;
    double cur_rl_ = 0;

    Clock::time_point stage_start_time_;

    ClientId client_id_ = 0;
    JobRefId registered_job_id_ = 0;
    void* remote_ptr_ = nullptr;
    JobId id_ = 0;
    JobId unique_id_ = 0;
};

}  // namespace job
}  // namespace llis
