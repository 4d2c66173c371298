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
// one message is sent per noti_batch_size workgroups plus one for the remainder, so a grid of n workgroups
// produces exactly ceil(n/batch) start messages and ceil(n/batch) end messages whose `num` fields sum to n
// (reference include/llis/job/finished_block_notifier.h:18-94, alloc at src/job/finished_block_notifier.cu:21-46).
//
// Ordering on gfx950: a workgroup's results must be visible to a kernel that the scheduler launches on a
// different stream as soon as the host has seen the end message.  Each workgroup therefore issues a
// device-scope release before it bumps the end counter, the sender acquires at device scope after the
// bump, and the message itself is a system-scope release store.
//
// Per-workgroup timing (optional, switched on when the array is created with a second ring): lane (0,0,0)
// samples the 100 MHz wall clock on entry and on exit and sends both, 24 bits each, as one BlockStartEndTime
// slot (reference LLIS_MEASURE_BLOCK_TIME, include/llis/job/finished_block_notifier.h:20-25,58-63,90-92; there a
// compile-time switch, one sample pair shared by all workgroups of a kernel, SM clock / 256).  The entry
// sample lives in LDS, so every workgroup reports its own pair; unit here: 10 ns.

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/instrument_info.h>

namespace llis {
namespace job {

class FinishedBlockNotifier {
  public:
    // Workgroups per message: a property of each notifier, fixed when it is created (create_array), a power of two
    // of at most 128 (`num` travels in one byte).  The reference batches 16 on a 40-SM GPU (reference
    // include/llis/job/finished_block_notifier.h:118) and that value is reference_noti_batch_size; the default,
    // 64, keeps a comparable share of a 256-CU device per message and quarters the host's message rate.  Grids of
    // up to 16 workgroups send exactly one start and one end message either way.
    static constexpr unsigned noti_batch_size = 64;
    static constexpr unsigned reference_noti_batch_size = 16;
    static constexpr unsigned max_noti_batch_size = 128;

    static constexpr bool valid_batch_size(unsigned b) { return b != 0 && b <= max_noti_batch_size && (b & (b - 1)) == 0; }

    FinishedBlockNotifier() {}
    explicit FinishedBlockNotifier(ipc::Gpu2SchedChannel* gpu2sched_channel, ipc::Gpu2SchedChannel* block_time_channel = nullptr,
                                   unsigned batch_size = noti_batch_size) {
        gpu2sched_channel_ = gpu2sched_channel->fork();
        if (block_time_channel) {
            block_time_channel_ = block_time_channel->fork();
            measure_block_time_ = 1;
        }
        batch_mask_ = (valid_batch_size(batch_size) ? batch_size : noti_batch_size) - 1;
    }
    FinishedBlockNotifier(FinishedBlockNotifier&&) = default;
    FinishedBlockNotifier& operator=(FinishedBlockNotifier&&) = default;

#if defined(__HIPCC__)
    __device__ __forceinline__ void start(JobId job_id) { start(job_id, gridDim.x * gridDim.y * gridDim.z); }

    // For a launch that carries the kernels of several jobs, each with a notifier of its own: `num_blocks` is the number
    // of workgroups of the launch that report to THIS notifier (the same value in start and end calls of one kernel).
    __device__ __forceinline__ void start(JobId job_id, unsigned num_blocks) {
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            if (measure_block_time_) *entry_clock_slot() = (unsigned)wall_clock64() & 0xFFFFFFu;
            announce<false>(&agg_counter_start_, 1, job_id, num_blocks);
        }
    }

    // For kernels that skip start() (no start message wanted) and were told by their caller that timing is on:
    // takes the entry sample without looking at the notifier.
    __device__ __forceinline__ void begin_timing() {
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) *entry_clock_slot() = (unsigned)wall_clock64() & 0xFFFFFFu;
    }

    // For arbitrary kernels: makes everything the workgroup wrote visible device-wide (cache write-back)
    // before the end message can be seen.
    __device__ __forceinline__ void end(JobId job_id) {
        __syncthreads();
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            if (measure_block_time_) send_block_time_first();
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
            if (measure_block_time_) send_block_time_first();
            announce<false>(&agg_counter_end_, 0, job_id);
        }
    }

    // Same, for callers that know from elsewhere whether timing is on (the flag is then not read here).
    __device__ __forceinline__ void end_written_through(JobId job_id, bool timed) {
        end_written_through(job_id, timed, gridDim.x * gridDim.y * gridDim.z);
    }
    // ... and how many workgroups of the launch report to this notifier (a launch that carries several jobs' kernels).
    __device__ __forceinline__ void end_written_through(JobId job_id, bool timed, unsigned num_blocks) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
            if (timed && timing_is_on()) send_block_time_first();  // the member is looked at only when timing was asked for
            announce<false>(&agg_counter_end_, 0, job_id, num_blocks);
        }
    }

    // The same again for kernels that find out by themselves when every wave of the workgroup has had its write-through
    // stores acknowledged (say, by counting waves in LDS): the ONE lane that establishes it calls this, no barrier is
    // involved, and the other waves may have left the compute unit already.
    __device__ __forceinline__ void end_from_one_lane(JobId job_id, bool timed) {
        end_from_one_lane(job_id, timed, gridDim.x * gridDim.y * gridDim.z);
    }
    __device__ __forceinline__ void end_from_one_lane(JobId job_id, bool timed, unsigned num_blocks) {
        if (timed && timing_is_on()) send_block_time_first();
        announce<false>(&agg_counter_end_, 0, job_id, num_blocks);
    }
#endif

    // Allocates `num` notifiers in device memory, all bound to the given ring (and, when given, to the ring
    // that receives per-workgroup timing samples), sending one message per `batch_size` workgroups; a batch size
    // that is no power of two in 1..128 is an error (std::invalid_argument).
    static FinishedBlockNotifier* create_array(unsigned num, ipc::Gpu2SchedChannel* gpu2sched_channel,
                                               ipc::Gpu2SchedChannel* block_time_channel = nullptr,
                                               unsigned batch_size = noti_batch_size);
    static void free_array(FinishedBlockNotifier* ptr);

  private:
#if defined(__HIPCC__)
    // One word of LDS per kernel that carries the hooks: the workgroup's entry sample (only lane (0,0,0) touches it).
    __device__ __forceinline__ static unsigned* entry_clock_slot() {
        __shared__ unsigned entry_clock;
        return &entry_clock;
    }

    // The flag through a volatile access: an ordinary load is hoisted above the test of `timed`, and a workgroup that was not
    // asked for timing then waits for a trip to memory of its own before it may count itself in.
    __device__ __forceinline__ bool timing_is_on() const { return *const_cast<const volatile unsigned*>(&measure_block_time_) != 0; }

    __device__ __forceinline__ void send_block_time() {
        const unsigned s = *entry_clock_slot();
        const unsigned e = (unsigned)wall_clock64() & 0xFFFFFFu;
        BlockStartEndTime t;  // 24 + 24 bits packed as in reference src/server/scheduler_full3.cpp:113-119
        t.data[0] = (uint16_t)(s >> 8);
        t.data[1] = (uint16_t)(((s & 0xFFu) << 8) | (e >> 16));
        t.data[2] = (uint16_t)(e & 0xFFFFu);
        block_time_channel_.write_relaxed(t);
    }

    // The workgroup's time sample goes out ahead of its end message, with a system-scope release between the two: once the
    // host has seen a kernel's last end message, every sample of that kernel is in the timing ring (a recording that stops
    // when the server is idle then holds whole kernels).  Only when per-workgroup timing is on.
    __device__ __forceinline__ void send_block_time_first() {
        send_block_time();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    }

    // ACQUIRE: the sender first acquires (device scope) what the other workgroups released before their bump.
    template <bool ACQUIRE>
    __device__ __forceinline__ void announce(unsigned* counter, uint8_t is_start, JobId job_id) {
        announce<ACQUIRE>(counter, is_start, job_id, gridDim.x * gridDim.y * gridDim.z);
    }
    template <bool ACQUIRE>
    __device__ __forceinline__ void announce(unsigned* counter, uint8_t is_start, JobId job_id, const unsigned num_blocks) {
        const unsigned mask = batch_mask_;  // requested before the atomic, so the two trips to memory overlap
        const unsigned total = atomicInc(counter, num_blocks - 1) + 1;  // wraps to 0 after the last block
        const unsigned in_batch = total & mask;
        unsigned covered = 0;
        if (in_batch == 0) {
            covered = mask + 1;
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

    // Read-only after creation ...
    ipc::Gpu2SchedChannel gpu2sched_channel_;
    ipc::Gpu2SchedChannel block_time_channel_;
    unsigned measure_block_time_ = 0;
    unsigned batch_mask_ = noti_batch_size - 1;
    // ... and, on a cache line of their own, the counters every workgroup bumps atomically: a load of the
    // fields above must not queue behind those atomics.
    alignas(128) unsigned agg_counter_start_ = 0;
    unsigned agg_counter_end_ = 0;
};

}  // namespace job
}  // namespace llis
