// Job definitions for the scripted device (tests only).  They have the same stage structure as the real
// jobs but "launch" by telling the test double how many workgroups the kernel has.
//   FAKE_VARIANT 0  fake_short : 10 kernels of 5 x 256, 32 regs, pre-notify on the last  (shape of dummy_short)
//   FAKE_VARIANT 1  fake_long  : 50 kernels of 5 x 256                                   (shape of dummy_long)
//   FAKE_VARIANT 2  fake_mem3  : copy, kernels of 40 / 200 / 17 workgroups with distinct footprints, copy(pre-notify)
//   FAKE_VARIANT 3  fake_big   : 3 kernels of 3000 x 256 x 64 regs -- never fits beside anything (over-subscription path)
//   FAKE_VARIANT 4  fake_self  : a copy stage that reports its own completion (from a thread of its own after 300 us when
//                                FAKE_SELF_THREAD=1, else before it returns), copy, kernel of 40, copy(pre-notify); output = input + 1
//   FAKE_VARIANT 5  fake_flaky : fake_mem3 whose every FAKE_FLAKY_EVERY-th run (counted over the process) answers with one wrong byte
//   FAKE_VARIANT 6  fake_raw   : kernels of 40 and 300 workgroups with un-aggregated hooks, one of 17 with aggregated hooks, one of 500
//                                with un-aggregated hooks (pre-notify)

#include <llis/job/context.h>
#include <llis/job/coroutine_job.h>

#include "paella_hip.h"

#include <cstdlib>
#include <cstring>
#include <thread>

#include <unistd.h>

extern "C" int fake_hip_kernel_launch(void* stream, uint32_t job_id, unsigned nblocks);
extern "C" int fake_hip_raw_kernel_launch(void* stream, uint32_t job_id, unsigned nblocks);

#ifndef FAKE_VARIANT
#error "define FAKE_VARIANT"
#endif

namespace {

class FakeJob : public llis::job::CoroutineJob {
  public:
    size_t get_input_size() override { return FAKE_VARIANT == 2 || FAKE_VARIANT == 4 || FAKE_VARIANT == 5 ? 100 : 5; }
    size_t get_output_size() override { return FAKE_VARIANT == 2 || FAKE_VARIANT == 4 || FAKE_VARIANT == 5 ? 100 : 11; }
    size_t get_param_size() override { return 4; }

    void one_time_init() override {}

    void kernel(unsigned blocks, unsigned threads, unsigned smem, unsigned regs, bool pre_notify) {
        unset_is_mem();
        set_num_blocks(blocks);
        set_num_threads_per_block(threads);
        set_smem_size_per_block(smem);
        set_num_registers_per_thread(regs);
        if (pre_notify) set_pre_notify();
        yield();
        (void)get_finished_block_notifier();  // a real kernel with aggregated hooks takes it as an argument
        fake_hip_kernel_launch(reinterpret_cast<void*>(get_cuda_stream()), get_id(), blocks);
    }

    void raw_kernel(unsigned blocks, unsigned threads, unsigned smem, unsigned regs, bool pre_notify) {
        unset_is_mem();
        set_num_blocks(blocks);
        set_num_threads_per_block(threads);
        set_smem_size_per_block(smem);
        set_num_registers_per_thread(regs);
        if (pre_notify) set_pre_notify();
        yield();
        fake_hip_raw_kernel_launch(reinterpret_cast<void*>(get_cuda_stream()), get_id(), blocks);
    }

    void body(void* io_ptr) override {
#if FAKE_VARIANT == 0 || FAKE_VARIANT == 1
        const int n = FAKE_VARIANT == 0 ? 10 : 50;
        for (int i = 0; i < n; ++i) kernel(5, 256, 0, 32, i == n - 1);
#elif FAKE_VARIANT == 2 || FAKE_VARIANT == 5
        set_is_mem();
        yield();
        llis_hip_memcpy_async(buf_, io_ptr, 100, LLIS_HIP_H2D, reinterpret_cast<void*>(get_cuda_stream()));
        kernel(40, 128, 1024, 64, false);
        kernel(200, 64, 0, 32, false);
        kernel(17, 256, 8192, 128, false);
        for (int i = 0; i < 100; ++i) buf_[i] = (char)(buf_[i] + 1);
#if FAKE_VARIANT == 5
        {
            static unsigned runs = 0;
            const char* every = std::getenv("FAKE_FLAKY_EVERY");
            const unsigned n = every ? (unsigned)std::atoi(every) : 0;
            if (n && ++runs % n == 0) buf_[7] = (char)(buf_[7] + 1);
        }
#endif
        set_is_mem();
        set_pre_notify();
        yield();
        llis_hip_memcpy_async(reinterpret_cast<char*>(io_ptr) + 100, buf_, 100, LLIS_HIP_D2H, reinterpret_cast<void*>(get_cuda_stream()));
#elif FAKE_VARIANT == 4
        set_is_mem();
        set_completes_itself();
        yield();
        {
            const char* threaded = std::getenv("FAKE_SELF_THREAD");
            llis::job::Job* self = this;
            char* stage = stage_;
            if (threaded && threaded[0] == '1') {
                std::thread([self, stage, io_ptr] {
                    usleep(300);
                    std::memcpy(stage, io_ptr, 100);
                    llis::job::Context::post_mem_completion(self);
                }).detach();
            } else {
                std::memcpy(stage, io_ptr, 100);
                llis::job::Context::post_mem_completion(self);
            }
        }
        unset_completes_itself();
        yield();
        llis_hip_memcpy_async(buf_, stage_, 100, LLIS_HIP_H2D, reinterpret_cast<void*>(get_cuda_stream()));
        kernel(40, 128, 1024, 64, false);
        for (int i = 0; i < 100; ++i) buf_[i] = (char)(buf_[i] + 1);
        set_is_mem();
        set_pre_notify();
        yield();
        llis_hip_memcpy_async(reinterpret_cast<char*>(io_ptr) + 100, buf_, 100, LLIS_HIP_D2H, reinterpret_cast<void*>(get_cuda_stream()));
#elif FAKE_VARIANT == 6
        raw_kernel(40, 256, 0, 32, false);
        raw_kernel(300, 64, 2048, 64, false);
        kernel(17, 256, 8192, 128, false);
        raw_kernel(500, 256, 0, 32, true);
#else
        for (int i = 0; i < 3; ++i) kernel(3000, 256, 0, 64, i == 2);
#endif
        (void)io_ptr;
    }

  private:
    char buf_[100];
    char stage_[100];
};

}  // namespace

extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new FakeJob(); }
