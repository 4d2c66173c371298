// vec_add_coroutine: a copy-in stage, ten vector-add kernels of 200 workgroups x 10 threads, a copy-out
// stage that wakes the client.  Output = 10 x input.  Stage sequence follows reference
// jobs/vec_add_coroutine/vec_add_coroutine.cu:8-141; unlike the reference the kernels work on device
// buffers and the copies go through runtime-pinned staging memory, because the client's request pool is
// ordinary shared memory that the GPU cannot address here.

#include <llis/job/context.h>
#include <llis/job/coroutine_job.h>

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace {

__global__ void vec_add(float* output, const float* input, size_t count, llis::JobId job_id, llis::job::FinishedBlockNotifier* notifier) {
    notifier->start(job_id);
    const unsigned stride = blockDim.x * gridDim.x;
    for (unsigned id = blockIdx.x * blockDim.x + threadIdx.x; id < count; id += stride) output[id] += input[id];
    notifier->end(job_id);
}

#define VA_CHECK(expr)                                                                    \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "vec_add job: %s failed: %s\n", #expr, hipGetErrorString(e_)); \
            std::abort();                                                                 \
        }                                                                                 \
    } while (0)

class VecAddCoroutineJob : public llis::job::CoroutineJob {
    static constexpr unsigned kCount = 32000;
    static constexpr unsigned kBlocks = 200;
    static constexpr unsigned kThreads = 10;
    static constexpr int kIters = 10;

  public:
    size_t get_input_size() override { return kCount * sizeof(float); }
    size_t get_output_size() override { return kCount * sizeof(float); }
    size_t get_param_size() override { return 4; }

    void one_time_init() override {
        set_num_threads_per_block(kThreads);
        set_num_blocks(kBlocks);
        set_smem_size_per_block(0);
        hipFuncAttributes attr;
        VA_CHECK(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(vec_add)));
        set_num_registers_per_thread((unsigned)attr.numRegs);
        VA_CHECK(hipMalloc(&input_dev_, get_input_size()));
        VA_CHECK(hipMalloc(&output_dev_, get_output_size()));
        VA_CHECK(hipHostMalloc(&staging_, get_input_size() + get_output_size(), hipHostMallocDefault));
    }

    void body(void* io_ptr) override {
        io_ptr_ = io_ptr;
        set_is_mem();
        yield();
        std::memcpy(staging_, io_ptr, get_input_size());
        VA_CHECK(hipMemcpyAsync(input_dev_, staging_, get_input_size(), hipMemcpyHostToDevice, get_cuda_stream()));
        VA_CHECK(hipMemsetAsync(output_dev_, 0, get_output_size(), get_cuda_stream()));
        unset_is_mem();

        for (int i = 0; i < kIters; ++i) {
            yield();
            hipLaunchKernelGGL(vec_add, dim3(kBlocks), dim3(kThreads), 0, get_cuda_stream(), output_dev_, input_dev_, (size_t)kCount, get_id(),
                               get_finished_block_notifier());
        }

        set_is_mem();
        set_pre_notify();
        yield();
        VA_CHECK(hipMemcpyAsync(staging_ + get_input_size(), output_dev_, get_output_size(), hipMemcpyDeviceToHost, get_cuda_stream()));
    }

    void on_complete() override { std::memcpy(reinterpret_cast<char*>(io_ptr_) + get_input_size(), staging_ + get_input_size(), get_output_size()); }

  private:
    float* input_dev_ = nullptr;
    float* output_dev_ = nullptr;
    char* staging_ = nullptr;
    void* io_ptr_ = nullptr;
};

}  // namespace

extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new VecAddCoroutineJob(); }
