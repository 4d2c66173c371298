#pragma once
// ModelJob -- the job definition shared by the model adapters: copy the request in, run the model one
// operator per scheduler stage, copy the result out and wake the client.  It has the shape of the
// reference's TVM adapters (reference jobs/tvm_mnist/tvm_mnist.cpp:10-64): same sizes, same stage
// sequence mem -> kernels -> mem(pre-notify), same extern "C" init_job entry point; the kernels come from
// the executor in paella_models.h instead of a TVM module.
//
// Differences, on purpose:
//  * the device-to-host stage copies the model OUTPUT (the reference copies its input buffer back);
//  * PAELLA_INPUT_RESIDENT=1 (measurement only) drops the host-to-device stage: the input stays in device memory;
//  * a tensor of at most PAELLA_ZERO_COPY_BYTES (default 64 KiB) gets no copy stage: the first kernel reads the input
//    from, the last kernel writes the output to, the pinned staging buffer across PCIe (the small CNN then has 5 stages
//    instead of 7, ResNet-18 no device-to-host stage); pre-notify moves to the last kernel;
//  * a model whose kernels all have at most PAELLA_GROUP_THREADS work-items (default 65536, an eighth of what the device
//    holds; 0 = off) is one scheduler stage: its kernels are issued together, in order on one queue, and only the last
//    one reports to the scheduler.  Scheduling kernel by kernel pays off for kernels that fill the device; for the small
//    CNN (5 kernels of at most 25 workgroups) each trip through the scheduler costs more than the kernel;
//  * request buffers in the client's shared-memory pool cannot be registered with the runtime on this
//    platform, so both copies go through a per-instance pinned staging buffer (filled on the server
//    thread just before the H2D copy is issued -- or, under a stage-by-stage scheduler, by a helper thread as a copy stage
//    of its own -- and drained in on_complete());
//  * under a scheduler that issues a whole job at once (fifo), PAELLA_DISPATCH=direct puts the job's kernels, in order, on one
//    of the operator library's direct-dispatch queues with the barrier bit set (a queue then behaves like a stream), the
//    input upload being a copy kernel on the same queue: plain per-request stream serving on the same launch path as the
//    stage-by-stage schedulers, so that a comparison with them is one of policy and not of launch cost.  Default there: HIP
//    streams and launches.

#include <llis/job/context.h>
#include <llis/job/coroutine_job.h>

#include "paella_hip.h"
#include "paella_models.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace paella {

class ModelJob : public llis::job::CoroutineJob {
  public:
    // onnx_stem: file name (without ".onnx") of the model's ONNX zoo file.  If $LLIS_MODELS_DIR/<stem>.onnx is readable
    // the adapter serves that file -- its graph and trained weights -- instead of the built-in seeded model; the
    // reference looks in the same directory for "<stem>-cuda_llis-pack.so" (reference jobs/tvm_mnist/tvm_mnist.cpp:27).
    explicit ModelJob(const char* model_name, const char* onnx_stem = nullptr) : name_(resolve(model_name, onnx_stem)) {
        if (paella_model_io_bytes(name_.c_str(), &in_bytes_, &out_bytes_) != 0) throw std::invalid_argument("cannot load model " + name_);
    }

    static std::string resolve(const char* model_name, const char* onnx_stem) {
        const char* dir = std::getenv("LLIS_MODELS_DIR");
        if (dir && *dir && onnx_stem) {
            const std::string path = std::string(dir) + "/" + onnx_stem + ".onnx";
            if (FILE* f = std::fopen(path.c_str(), "rb")) {
                std::fclose(f);
                return "onnx:" + path;
            }
        }
        return model_name;
    }

    size_t get_input_size() override { return in_bytes_; }
    size_t get_output_size() override { return out_bytes_; }
    size_t get_param_size() override { return 4; }

    void one_time_init() override {
        const char* seed_env = std::getenv("LLIS_MODEL_SEED");
        const uint64_t seed = seed_env ? std::strtoull(seed_env, nullptr, 10) : 1;
        check(paella_model_get(name_.c_str(), seed, &model_), "paella_model_get");
        check(paella_exec_create(model_, &exec_), "paella_exec_create");
        void* p = nullptr;
        out_off_ = (in_bytes_ + 255) / 256 * 256;
        check(llis_hip_host_alloc_pinned(&p, out_off_ + out_bytes_), "pinned staging");
        staging_ = reinterpret_cast<char*>(p);
        num_stages_ = paella_model_num_stages(model_);
        const char* grp = std::getenv("PAELLA_GROUP_THREADS");
        const unsigned long group_limit = grp ? std::strtoul(grp, nullptr, 10) : 65536;
        // Only a model made of small kernels throughout is issued in one piece.  Grouping the small kernels of a large
        // model (ResNet-18's projections and its global pool) was measured too: 13.9 -> 12.8 k requests/s at saturation,
        // because a member that must wait for its predecessor stalls everything behind it in its queue.
        bool all_small = group_limit > 0;
        for (int s = 0; s < num_stages_ && all_small; ++s) {
            paella_launch_dims d;
            paella_model_stage_dims(model_, s, &d);
            all_small = (unsigned long)d.grid * d.block <= group_limit;
        }
        group_end_.assign((size_t)num_stages_, 0);
        for (int s = 0; s < num_stages_; ++s) group_end_[(size_t)s] = all_small ? num_stages_ - 1 : s;
        // Kernels go out as AQL packets on the operator library's own queues unless PAELLA_DISPATCH=hip; the
        // copies stay on the pooled HIP stream.  Only under a scheduler that orders a job's stages through the
        // notification ring (fifo2, full3): the queues have no ordering of their own, and fifo relies on the stream.
        const char* resident = std::getenv("PAELLA_INPUT_RESIDENT");
        input_resident_ = resident && std::strcmp(resident, "1") == 0;
        const char* zc = std::getenv("PAELLA_ZERO_COPY_BYTES");
        const size_t zero_copy_limit = zc ? std::strtoull(zc, nullptr, 10) : 65536;
        zero_in_ = !input_resident_ && in_bytes_ <= zero_copy_limit && paella_exec_bind_input(exec_, staging_) == 0;
        zero_out_ = out_bytes_ <= zero_copy_limit && paella_exec_bind_output(exec_, staging_ + out_off_) == 0;
        timed_ = llis::job::Context::get_gpu2sched_block_time_channel()->is_connected();  // server runs with --measure_block_time
        const char* starts = std::getenv("PAELLA_UNFIT_STARTS");
        unfit_starts_ = starts && std::strcmp(starts, "1") == 0;
        const char* dispatch = std::getenv("PAELLA_DISPATCH");
        direct_ = !(dispatch && std::strcmp(dispatch, "hip") == 0) && llis::job::Context::is_stage_by_stage();
        // whole-job issue on an ordered direct queue: asked for by name, and only when no copy has to stay on the HIP stream
        // behind the kernels (every model's output here is small enough to be written by its last kernel)
        whole_job_direct_ = !llis::job::Context::is_stage_by_stage() && dispatch && std::strcmp(dispatch, "direct") == 0 && zero_out_ &&
                            in_bytes_ % sizeof(float) == 0;
        if (direct_ || whole_job_direct_) {
            void* probe = nullptr;
            if (paella_direct_queue_shared(&probe) != 0) {
                std::fprintf(stderr, "[llis] model job: direct dispatch unavailable, using HIP launches\n");
                direct_ = whole_job_direct_ = false;
            }
        }
        // Conv launches of different requests share launches (paella_pack_enable) unless PAELLA_PACK=0: the serving thread
        // holds them and lets them go from its loop.
        const char* pack = std::getenv("PAELLA_PACK");
        pack_ = direct_ && !(pack && std::strcmp(pack, "0") == 0);
        if (pack_) llis::job::Context::add_poll_hook(&paella_pack_poll_hook);  // one address for every adapter library: registered once
        // The staging copy of an input too large for zero-copy leaves the serving thread unless PAELLA_STAGE_THREAD=0; only
        // under a scheduler that waits for a stage's completion before it issues the next one.
        const char* st = std::getenv("PAELLA_STAGE_THREAD");
        stage_off_thread_ = llis::job::Context::is_stage_by_stage() && !(st && std::strcmp(st, "0") == 0);
    }

    void body(void* io_ptr) override {
        io_ptr_ = io_ptr;
        if (zero_in_) {
            // no stage of its own: staged just before the first kernel is issued, below
        } else if (!input_resident_) {
            set_is_mem();
            if (stage_off_thread_) {
                // The host-side copy into the staging buffer is a copy stage of its own, done by the operator library's helper
                // thread, which reports it to the scheduler like a finished copy: the serving thread keeps reading its rings.
                set_completes_itself();
                yield();
                const int rc = paella_host_copy_submit(staging_, io_ptr, in_bytes_, &ModelJob::staged, static_cast<llis::job::Job*>(this));
                if (rc == PAELLA_EBUSY) {  // the helper sleeps: a quiet moment, the copy is done here
                    std::memcpy(staging_, io_ptr, in_bytes_);
                    staged(static_cast<llis::job::Job*>(this));
                } else {
                    check(rc, "staging copy");
                }
                unset_completes_itself();
                yield();
            } else {
                yield();
                std::memcpy(staging_, io_ptr, in_bytes_);
            }
            if (whole_job_direct_) {
                // the upload as a kernel that reads the pinned staging buffer, first packet of this job on its queue (the
                // scheduler's completion marker for the copy stage goes to the idle HIP stream and counts at once; the job
                // ends when its last kernel's workgroups have reported)
                check(paella_direct_queue_shared(&job_queue_), "direct queue");
                paella_direct_queue_set_ordered(job_queue_, 1);
                check(paella_copy_launch(reinterpret_cast<const float*>(staging_), reinterpret_cast<float*>(paella_exec_input(exec_)),
                                         in_bytes_ / sizeof(float), job_queue_, 0, nullptr), "upload kernel");
            } else {
                check(llis_hip_memcpy_async(paella_exec_input(exec_), staging_, in_bytes_, LLIS_HIP_H2D, stream()), "H2D");
            }
            unset_is_mem();
        } else if (!input_uploaded_) {
            // Measurement mode PAELLA_INPUT_RESIDENT=1: the instance's input is uploaded once, from its first
            // request, and every request then runs kernels + the result copy only (no host-to-device stage).
            check(llis_hip_memcpy(paella_exec_input(exec_), io_ptr, in_bytes_, LLIS_HIP_H2D), "initial H2D");
            input_uploaded_ = true;
        }

        for (int s = 0; s < num_stages_;) {
            const int last = group_end_[(size_t)s];
            paella_launch_dims d;
            paella_model_stage_dims(model_, last, &d);  // the group is admitted and accounted as its last kernel
            set_num_blocks(d.grid);
            set_num_threads_per_block(d.block);
            set_smem_size_per_block(d.lds_bytes);
            set_num_registers_per_thread(d.vgprs);
            if (zero_out_ && last == num_stages_ - 1) set_pre_notify();
            yield();
            if (zero_in_ && s == 0) std::memcpy(staging_, io_ptr, in_bytes_);
            // Workgroup starts are reported only on request (PAELLA_UNFIT_STARTS=1), and then only by a kernel admitted beyond
            // the occupancy budget ("unfit"), whose over-subscription credit full3 returns once all its workgroups are resident;
            // without start messages the credit returns when the kernel ends (reference src/server/scheduler_full3.cpp:196-204).
            const uint32_t id = get_id() | (is_unfit() && unfit_starts_ ? 0u : PAELLA_JOB_ID_NO_START) | (timed_ ? PAELLA_JOB_ID_TIME_BLOCKS : 0u);
            void* target = stream();
            if (direct_) check(paella_direct_queue_shared(&target), "direct queue");
            if (whole_job_direct_) {
                if (!job_queue_) {  // no upload stage came first
                    check(paella_direct_queue_shared(&job_queue_), "direct queue");
                    paella_direct_queue_set_ordered(job_queue_, 1);
                }
                target = job_queue_;
            }
            if (pack_) enable_packing_on_this_thread();
            // members of a group wait for what is ahead of them in the queue (a stream orders by itself); the first one
            // too, so that it is not held back for packing while the others go out
            if (direct_ && last > s) paella_direct_queue_set_ordered(target, 1);
            // ... and the whole group is recorded, to go out together with the same group of other requests of this model
            const bool recording = pack_ && last > s && paella_pack_sequence_begin(model_, target) == 0;
            for (int k = s; k <= last; ++k) {
                if (k < last) check(paella_exec_launch_stage(exec_, k, target, 0, nullptr), "stage launch");
                else check(paella_exec_launch_stage(exec_, k, target, id, get_finished_block_notifier()), "stage launch");
            }
            if (recording) check(paella_pack_sequence_end(), "end of the recorded launch sequence");
            if (direct_ && last > s) paella_direct_queue_set_ordered(target, 0);
            s = last + 1;
        }
        if (job_queue_) {  // the whole job is out (the scheduler drained this coroutine in one go): the queue is the next job's
            paella_direct_queue_set_ordered(job_queue_, 0);
            job_queue_ = nullptr;
        }

        if (zero_out_) return;
        set_is_mem();
        set_pre_notify();
        yield();
        check(llis_hip_memcpy_async(staging_ + out_off_, paella_exec_output(exec_), out_bytes_, LLIS_HIP_D2H, stream()), "D2H");
    }

    // The output sits right after the input bytes of the request slot (what the client library reads).
    void on_complete() override { std::memcpy(reinterpret_cast<char*>(io_ptr_) + in_bytes_, staging_ + out_off_, out_bytes_); }

  private:
    void* stream() { return reinterpret_cast<void*>(get_cuda_stream()); }

    static void staged(void* job) { llis::job::Context::post_mem_completion(static_cast<llis::job::Job*>(job)); }

    // Packing is a property of the launching thread (the serving thread, which also runs pack_poll from its loop).
    static void enable_packing_on_this_thread() {
        static thread_local bool on = false;
        if (!on) {
            paella_pack_enable(1);
            on = true;
        }
    }

    static void check(int rc, const char* what) {
        if (rc != 0) {
            std::fprintf(stderr, "[llis] model job: %s failed: %d (%s)\n", what, rc, rc > 0 ? llis_hip_error_string(rc) : "bad argument");
            std::abort();
        }
    }

    std::string name_;
    size_t in_bytes_ = 0, out_bytes_ = 0, out_off_ = 0;
    paella_model* model_ = nullptr;
    paella_exec* exec_ = nullptr;
    char* staging_ = nullptr;
    void* io_ptr_ = nullptr;
    int num_stages_ = 0;
    std::vector<int> group_end_;   // per kernel: index of the last kernel of the group it is issued with
    bool direct_ = true;
    bool whole_job_direct_ = false;
    void* job_queue_ = nullptr;    // whole-job issue: the ordered queue this request's kernels are going to
    bool pack_ = false;
    bool stage_off_thread_ = false;
    bool timed_ = false;
    bool unfit_starts_ = false;
    bool input_resident_ = false, input_uploaded_ = false;
    bool zero_in_ = false, zero_out_ = false;
};

}  // namespace paella

#define PAELLA_DEFINE_MODEL_JOB(ClassName, model_name, onnx_stem)                                        \
    class ClassName : public paella::ModelJob {                                                          \
      public:                                                                                            \
        ClassName() : paella::ModelJob(model_name, onnx_stem) {}                                         \
    };                                                                                                   \
    extern "C" __attribute__((visibility("default"))) llis::job::Job* init_job() { return new ClassName(); }
