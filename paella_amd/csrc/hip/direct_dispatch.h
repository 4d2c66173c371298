#pragma once
// Direct dispatch: operator kernels submitted as AQL packets to user-mode hardware queues owned by this
// library, bypassing the HIP launch path (2.3 to 3.9 us of host time per launch on this platform, the largest
// cost of kernel-by-kernel scheduling).  A dispatch is: pack the kernel arguments into the queue's kernarg
// ring, fill one 64-byte packet, store its header, ring the doorbell -- a few hundred nanoseconds.
//
// Ordering and completion are the scheduler's business, as in the serving path: packets carry no barrier bit
// and no completion signal (kernels of different jobs that share a queue overlap; a job's next stage is only
// dispatched after its notifier reported the previous one).  Packets acquire at agent scope and do not
// release: the operator kernels write their results through to memory.  Kernel arguments live in device
// memory.
//
// The kernels are the same device code as the HIP path: each ops_*.hip file is also compiled to a plain code
// object that is embedded in the library and loaded through the HSA loader on first use.

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstring>

namespace paella {

struct DirectQueue;

struct DirectKernel {
    uint64_t object = 0;          // address of the kernel descriptor
    uint32_t kernarg_bytes = 0;   // explicit arguments + the 256-byte implicit block
    uint32_t static_lds = 0;
    uint32_t private_bytes = 0;
};

// Number of live direct queues; zero means every handle is a HIP stream (fast path of direct_queue_lookup).
extern int g_direct_queue_count;

// Returns the queue if `handle` is one created by direct_queue_create(), else nullptr.
DirectQueue* direct_queue_lookup_slow(void* handle);
inline DirectQueue* direct_queue_lookup(void* handle) { return g_direct_queue_count == 0 ? nullptr : direct_queue_lookup_slow(handle); }

// Resolves (and caches) the device kernel behind a host-side kernel function pointer.  Aborts with a message
// if the kernel is not in the embedded code objects.
const DirectKernel* direct_kernel(const void* host_function);

// `used_bytes` (0 = all): the kernel reads only that much of its explicit arguments (a group launch with fewer members than
// the argument block has room for); the rest of the block is not written.
void direct_dispatch(DirectQueue* queue, const DirectKernel* kernel, dim3 grid, dim3 block, unsigned dynamic_lds, const void* explicit_args,
                     size_t explicit_bytes, size_t used_bytes = 0);

// True while the queue puts the barrier bit on its packets (paella_direct_queue_set_ordered).
bool direct_queue_ordered(const DirectQueue* queue);

// Fewest packets waiting (written but not yet taken by the packet processor) on any queue of the shared set; 0 when
// there is no shared set yet.
uint64_t direct_shared_min_waiting();

// Kernel-argument packing: every argument at its natural alignment, in order (the kernarg segment layout of
// by-value arguments).
inline void pack_args(char*, size_t& offset) { (void)offset; }
template <typename T, typename... Rest>
inline void pack_args(char* buf, size_t& offset, const T& first, const Rest&... rest) {
    offset = (offset + alignof(T) - 1) & ~(alignof(T) - 1);
    std::memcpy(buf + offset, &first, sizeof(T));
    offset += sizeof(T);
    pack_args(buf, offset, rest...);
}

constexpr size_t kMaxExplicitArgBytes = 2304;  // largest: eight conv problems in one launch

// Clock bridge for latency probes: the host's reading of the system timestamp, its frequency, and the
// translation of a device realtime-counter value (what wall_clock64() returns in a kernel) into that domain.
// False if the runtime is unavailable.
bool direct_system_clock(uint64_t* now_ticks, uint64_t* ticks_per_second);
bool direct_device_tick_to_system(uint64_t device_tick, uint64_t* system_tick);

}  // namespace paella
