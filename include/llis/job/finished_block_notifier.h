#pragma once
// Device-resident object through which every compute kernel reports workgroup residency and completion.
//
//   __global__ void k(..., llis::JobId job_id, llis::job::FinishedBlockNotifier* notifier) {
//       notifier->start(job_id);      // first statement
//       ...
//       notifier->end(job_id);        // last statement, reached by ALL threads (contains a barrier)
//   }
//
// Aggregation: lane (0,0,0) of each workgroup bumps a per-notifier counter that wraps at the grid size;
// one message is sent per 16 workgroups plus one for the remainder, so a grid of n workgroups produces
// exactly ceil(n/16) start messages and ceil(n/16) end messages whose `num` fields sum to n
// (reference include/llis/job/finished_block_notifier.h:18-94, alloc at src/job/finished_block_notifier.cu:21-46).
//
// Ordering on gfx950: a workgroup's results must be visible to a kernel that the scheduler launches on a
// different stream as soon as the host has seen the end message.  Each workgroup therefore issues a
// device-scope release before it bumps the end counter, the sender acquires at device scope after the
// bump, and the message itself is a system-scope release store.

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/instrument_info.h>

namespace llis {
namespace job {

class FinishedBlockNotifier {
  public:
    // Workgroups per message.  The reference batches 16 on a 40-SM GPU (reference
    // include/llis/job/finished_block_notifier.h:118); 64 keeps a comparable share of a 256-CU device per
    // message and quarters the host's message rate.  Grids of up to 64 workgroups send exactly one start
    // and one end message either way.
    static constexpr unsigned noti_batch_size = 64;

    FinishedBlockNotifier() {}
    explicit FinishedBlockNotifier(ipc::Gpu2SchedChannel* gpu2sched_channel) {
        gpu2sched_channel_ = gpu2sched_channel->fork();
    }
    FinishedBlockNotifier(FinishedBlockNotifier&&) = default;
    FinishedBlockNotifier& operator=(FinishedBlockNotifier&&) = default;

#if defined(__HIPCC__)
    __device__ __forceinline__ void start(JobId job_id) {
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            announce<false>(&agg_counter_start_, 1, job_id);
        }
    }

    // For arbitrary kernels: makes everything the workgroup wrote visible device-wide (cache write-back)
    // before the end message can be seen.
    __device__ __forceinline__ void end(JobId job_id) {
        __syncthreads();
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            announce<true>(&agg_counter_end_, 0, job_id);
        }
    }

    // For kernels that wrote ALL their results with device-scope write-through stores
    // (__hip_atomic_store(..., __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)): every wave waits until its own
    // stores have been acknowledged, then the barrier; no cache write-back is needed, which keeps the
    // per-workgroup cost of the hook at one atomic.
    __device__ __forceinline__ void end_written_through(JobId job_id) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            announce<false>(&agg_counter_end_, 0, job_id);
        }
    }
#endif

    // Allocates `num` notifiers in device memory, all bound to the given ring.
    static FinishedBlockNotifier* create_array(unsigned num, ipc::Gpu2SchedChannel* gpu2sched_channel);
    static void free_array(FinishedBlockNotifier* ptr);

  private:
#if defined(__HIPCC__)
    // ACQUIRE: the sender first acquires (device scope) what the other workgroups released before their bump.
    template <bool ACQUIRE>
    __device__ __forceinline__ void announce(unsigned* counter, uint8_t is_start, JobId job_id) {
        const unsigned num_blocks = gridDim.x * gridDim.y * gridDim.z;
        const unsigned total = atomicInc(counter, num_blocks - 1) + 1;  // wraps to 0 after the last block
        const unsigned in_batch = total % noti_batch_size;
        unsigned covered = 0;
        if (in_batch == 0) {
            covered = noti_batch_size;
        } else if (total == num_blocks) {
            covered = in_batch;
        }
        if (covered != 0) {
            if (ACQUIRE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            InstrumentInfo info;
            info.is_start = is_start;
            info.num = (uint8_t)covered;
            info.job_id = job_id;
            // The counter chain already ordered every workgroup's data before this point.
            gpu2sched_channel_.write_relaxed(info);
        }
    }
#endif

    ipc::Gpu2SchedChannel gpu2sched_channel_;
    unsigned agg_counter_start_ = 0;
    unsigned agg_counter_end_ = 0;
};

}  // namespace job
}  // namespace llis
