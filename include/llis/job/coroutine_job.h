#pragma once
// CoroutineJob -- write a job as straight-line code that yields once per stage.
//
//   void body(void* io_ptr) override {
//       set_is_mem();  yield();  hipMemcpyAsync(..., get_cuda_stream());  unset_is_mem();
//       for (...) { set_num_blocks(...); ...; yield();  kernel<<<..., get_cuda_stream()>>>(..., get_id(), get_finished_block_notifier()); }
//       set_is_mem();  set_pre_notify();  yield();  hipMemcpyAsync(...);
//   }
//
// init() starts body() immediately and runs it up to its first yield(), because the scheduler needs the
// first stage's declaration before it can admit the job; every run_next() resumes it until the next
// yield() or the end of body().  Same surface and semantics as reference
// include/llis/job/coroutine_job.h:9-45; the stackful coroutine underneath is a private ~40-instruction
// x86-64 context switch (no Boost), with one lazily allocated, reused stack per job instance.

#include <llis/job/job.h>

namespace llis {
namespace job {

class CoroutineJob : public Job {
  public:
    CoroutineJob() {}
    ~CoroutineJob() override;
    CoroutineJob(const CoroutineJob&) = delete;
    CoroutineJob& operator=(const CoroutineJob&) = delete;

    void full_init(void* io_ptr) final {
        one_time_init();
        init(io_ptr);
    }

    void init(void* io_ptr) final;

    void run_next() final { resume(); }

    bool has_next() const final { return !finished_; }

    virtual void one_time_init() = 0;
    virtual void body(void* io_ptr) = 0;

    // Suspends body() and returns control to whoever called init()/run_next().
    void yield();

    static constexpr size_t kStackBytes = 256 * 1024;

  private:
    void resume();
    static void entry_trampoline();

    void* stack_base_ = nullptr;   // mmap'ed region: one guard page followed by kStackBytes
    void* coroutine_sp_ = nullptr; // saved stack pointer of the suspended body()
    void* caller_sp_ = nullptr;    // saved stack pointer of the resumer
    void* io_ptr_ = nullptr;
    bool finished_ = true;
};

}  // namespace job
}  // namespace llis
