// helloworld: a plain (non-coroutine) Job with five stages; stage i launches i workgroups of one thread
// that report through the un-aggregated kernel_start/kernel_end hooks, with the channel passed by value
// (reference jobs/helloworld/helloworld.cu:8-83).

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/context.h>
#include <llis/job/instrument.h>
#include <llis/job/job.h>

#include <hip/hip_runtime.h>

namespace {

__global__ void helloworld(int* sink, int i, llis::JobId job_id, llis::ipc::Gpu2SchedChannel gpu2sched_channel) {
    llis::job::kernel_start(job_id, &gpu2sched_channel);
    if (sink) atomicAdd(sink, i);
    llis::job::kernel_end(job_id, &gpu2sched_channel);
}

class HelloWorldJob : public llis::job::Job {
  public:
    size_t get_input_size() override { return 5; }
    size_t get_output_size() override { return 11; }
    size_t get_param_size() override { return 4; }

    void full_init(void* io_ptr) override {
        set_num_threads_per_block(1);
        set_smem_size_per_block(0);
        set_num_registers_per_thread(32);
        init(io_ptr);
    }

    void init(void*) override {
        num_ = 0;
        set_num_blocks(1);
    }

    void run_next() override {
        ++num_;
        hipLaunchKernelGGL(helloworld, dim3(num_), dim3(1), 0, get_cuda_stream(), (int*)nullptr, num_, get_id(),
                           llis::job::Context::get_gpu2sched_channel()->fork());
        set_num_blocks(num_ + 1);
        if (num_ == 4) set_pre_notify();  // the NEXT stage is the last one: wake the client when it is dispatched
    }

    bool has_next() const override { return num_ < 5; }

  private:
    int num_ = 0;
};

}  // namespace

extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new HelloWorldJob(); }
