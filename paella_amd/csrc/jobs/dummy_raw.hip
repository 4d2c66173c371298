// dummy_raw: three kernels of 64, 300 and 24 workgroups x 256 threads whose workgroups report one by one through the
// un-aggregated hooks (llis/job/instrument.h), naming the compute unit they run on -- the kind of job the
// per-compute-unit placement model reconciles its predictions with.  Each workgroup spins for a few microseconds so that
// the workgroups of a kernel are resident together.  The client is woken when the last kernel is dispatched.
// (The reference's only job with these hooks is jobs/helloworld/helloworld.cu, whose grids of 1..5 single-thread
// workgroups say nothing about placement.)

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/context.h>
#include <llis/job/coroutine_job.h>
#include <llis/job/instrument.h>

#include <hip/hip_runtime.h>

namespace {

__global__ void raw_kernel(unsigned spin_ticks, llis::JobId job_id, llis::ipc::Gpu2SchedChannel gpu2sched_channel) {
    llis::job::kernel_start(job_id, &gpu2sched_channel);
    const unsigned long long t0 = wall_clock64();   // 100 MHz
    while (wall_clock64() - t0 < spin_ticks) {
    }
    llis::job::kernel_end(job_id, &gpu2sched_channel);
}

class DummyRawJob : public llis::job::CoroutineJob {
  public:
    size_t get_input_size() override { return 5; }
    size_t get_output_size() override { return 11; }
    size_t get_param_size() override { return 4; }

    void one_time_init() override {
        set_num_threads_per_block(256);
        set_smem_size_per_block(0);
        set_num_registers_per_thread(32);
        unset_is_mem();
    }

    void body(void*) override {
        static const unsigned grids[3] = {64, 300, 24};
        for (int i = 0; i < 3; ++i) {
            set_num_blocks(grids[i]);
            if (i == 2) set_pre_notify();
            yield();
            hipLaunchKernelGGL(raw_kernel, dim3(grids[i]), dim3(256), 0, get_cuda_stream(), 2000u /* 20 us */, get_id(),
                               llis::job::Context::get_gpu2sched_channel()->fork());
        }
    }
};

}  // namespace

extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new DummyRawJob(); }
