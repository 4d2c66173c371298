#pragma once
// One launch helper for every operator kernel.  Normally a plain asynchronous launch; when the calling thread
// has armed a pair of timing events (paella_ops_time_launches) the launch goes through the runtime's extended
// entry point, which stamps the events with the kernel's own begin and end times on the device -- the same
// timestamps a kernel trace reports -- instead of the stream position before and after it.

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

namespace paella {

struct TimingEvents {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};

TimingEvents& timing_events();  // thread-local; defined in ops_misc.hip

template <typename Kernel, typename... Args>
inline void launch(Kernel kernel, dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream, Args... args) {
    const TimingEvents& t = timing_events();
    if (t.start != nullptr) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, t.start, t.stop, 0, args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args...);
    }
}

}  // namespace paella
