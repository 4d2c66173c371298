#pragma once
// One launch helper for every operator kernel.  Normally a plain asynchronous launch; when the calling thread
// has armed a pair of timing events (paella_ops_time_launches) the launch goes through the runtime's extended
// entry point, which stamps the events with the kernel's own begin and end times on the device -- the same
// timestamps a kernel trace reports -- instead of the stream position before and after it.  When the stream
// handle is a direct-dispatch queue the kernel goes out as an AQL packet instead (direct_dispatch.h).

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include "direct_dispatch.h"
#include "pack.h"

namespace paella {

struct TimingEvents {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};

TimingEvents& timing_events();  // thread-local; defined in ops_misc.hip

// `used_bytes` (0 = all): how much of the argument block the kernel reads (see direct_dispatch).
template <typename Kernel, typename... Args>
inline void launch_used(Kernel kernel, dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream, size_t used_bytes, const Args&... args) {
    pack_sequence_break();  // a launch that the sequence recorder did not take ends the recording (see pack.h)
    // `stream` is either a HIP stream or a direct-dispatch queue (paella_direct_queue_create).
    if (DirectQueue* q = direct_queue_lookup(reinterpret_cast<void*>(stream))) {
        alignas(16) char buf[kMaxExplicitArgBytes];
        size_t bytes = 0;
        static_assert((0 + ... + (sizeof(Args) + alignof(Args))) <= kMaxExplicitArgBytes, "kernel arguments do not fit the staging buffer");
        pack_args(buf, bytes, args...);
        direct_dispatch(q, direct_kernel(reinterpret_cast<const void*>(kernel)), grid, block, lds_bytes, buf, bytes, used_bytes);
        return;
    }
    const TimingEvents& t = timing_events();
    if (t.start != nullptr) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, t.start, t.stop, 0, args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args...);
    }
}

template <typename Kernel, typename... Args>
inline void launch(Kernel kernel, dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream, const Args&... args) {
    launch_used(kernel, grid, block, lds_bytes, stream, 0, args...);
}

}  // namespace paella
