#pragma once
// Synthetic fixed-shape job used for fairness and scheduling-order experiments: N identical kernels of
// 5 workgroups x 256 threads, each writing 100! (as a float product) over a 5,000,000-element buffer with
// a grid-stride loop; no copy stages; the client is woken when the last kernel is dispatched.
// Shape, sizes and stage sequence follow reference jobs/dummy_long/dummy_long.cu:8-78 (N = 50) and
// jobs/dummy_short/dummy_short.cu, jobs/dummy_10|11|20|21/dummy.cu (N = 10, 10, 11, 20, 21).
//
// Each job library defines DUMMY_NUM_KERNELS and includes this file.

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/context.h>
#include <llis/job/coroutine_job.h>
#include <llis/job/instrument.h>

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#ifndef DUMMY_NUM_KERNELS
#error "define DUMMY_NUM_KERNELS before including dummy_common.h"
#endif

namespace {

__global__ void dummy_kernel(float* mem, unsigned count, unsigned compute_count, llis::JobId job_id,
                             llis::job::FinishedBlockNotifier* notifier) {
    notifier->start(job_id);

    const unsigned stride = blockDim.x * gridDim.x;
    for (unsigned id = blockIdx.x * blockDim.x + threadIdx.x; id < count; id += stride) {
        float v = 1;
        for (unsigned i = 1; i <= compute_count; ++i) v *= i;
        mem[id] = v;
    }

    notifier->end(job_id);
}

class DummyCoroutineJob : public llis::job::CoroutineJob {
  public:
    size_t get_input_size() override { return 5; }
    size_t get_output_size() override { return 11; }
    size_t get_param_size() override { return 4; }

    void one_time_init() override {
        set_num_threads_per_block(256);
        set_smem_size_per_block(0);
        set_num_registers_per_thread(32);
        set_num_blocks(5);
        unset_is_mem();
        if (hipMalloc(&mem_, kCount * sizeof(float)) != hipSuccess) {
            std::fprintf(stderr, "dummy job: device allocation failed\n");
            std::abort();
        }
    }

    void body(void*) override {
        for (int i = 0; i < DUMMY_NUM_KERNELS; ++i) {
            if (i == DUMMY_NUM_KERNELS - 1) set_pre_notify();
            yield();
            hipLaunchKernelGGL(dummy_kernel, dim3(get_num_blocks()), dim3(get_num_threads_per_block()), 0, get_cuda_stream(), mem_, kCount,
                               kComputeCount, get_id(), get_finished_block_notifier());
        }
    }

  private:
    static constexpr unsigned kCount = 5000000;
    static constexpr unsigned kComputeCount = 100;
    float* mem_ = nullptr;
};

}  // namespace

extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new DummyCoroutineJob(); }
