// Implementation of the thin C-ABI over the HIP runtime declared in include/paella_hip.h.

#include <hip/hip_runtime.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "paella_hip.h"

namespace {

// HIP multiplexes streams onto a small number of hardware queues (4 by default) and kernels that share a
// queue run one after another, which caps how many requests can overlap on the GPU.  The block-level
// scheduler relies on real concurrency between streams, so unless the user chose a value the library asks
// for 16 queues before the runtime initialises (measured: 4 -> 16 queues raises served requests/s by ~30 %;
// 32 is slower again).
__attribute__((constructor)) void request_hardware_queues() { setenv("GPU_MAX_HW_QUEUES", "16", /*overwrite=*/0); }

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t value, size_t count) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) dst[i] = value;
}

// One lane claims a ring slot (device-scope wrapping increment) and publishes the message with a
// system-scope release store; stream order guarantees the preceding copy has completed.
__global__ void ring_marker_kernel(uint64_t* slots, unsigned last, unsigned* cursor, uint64_t message) {
    const unsigned pos = atomicInc(cursor, last);
    __hip_atomic_store(slots + pos, message, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

inline hipStream_t S(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline hipEvent_t E(void* e) { return reinterpret_cast<hipEvent_t>(e); }

hipMemcpyKind kind_of(int kind) {
    switch (kind) {
        case LLIS_HIP_H2D: return hipMemcpyHostToDevice;
        case LLIS_HIP_D2H: return hipMemcpyDeviceToHost;
        case LLIS_HIP_D2D: return hipMemcpyDeviceToDevice;
        default: return hipMemcpyDefault;
    }
}

}  // namespace

extern "C" {

int llis_hip_device_count(int* count) { return (int)hipGetDeviceCount(count); }

int llis_hip_set_device(int device) { return (int)hipSetDevice(device); }

int llis_hip_get_device_caps(llis_hip_device_caps* caps) {
    if (!caps) return (int)hipErrorInvalidValue;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    std::memset(caps, 0, sizeof(*caps));
    caps->num_cus = prop.multiProcessorCount;
    caps->wavefront_size = prop.warpSize;
    caps->max_threads_per_cu = prop.maxThreadsPerMultiProcessor;
    // The runtime's properties carry CUDA-shaped figures here (65536 "registers per multiprocessor", 2 "blocks per
    // multiprocessor"); a gfx950 compute unit has 4 SIMDs of 512 vector registers x 64 lanes and one workgroup slot per
    // wave slot.
    caps->max_blocks_per_cu = prop.maxThreadsPerMultiProcessor / prop.warpSize;
    caps->vgprs_per_cu = 4 * 512 * prop.warpSize;
    caps->lds_bytes_per_cu = (int)(prop.maxSharedMemoryPerMultiProcessor > 0 ? prop.maxSharedMemoryPerMultiProcessor
                                                                             : prop.sharedMemPerBlock);
    caps->clock_khz = prop.clockRate;
    caps->l2_bytes = prop.l2CacheSize;
    std::snprintf(caps->name, sizeof(caps->name), "%s", prop.gcnArchName);
    return 0;
}

const char* llis_hip_error_string(int code) { return hipGetErrorString((hipError_t)code); }

int llis_hip_stream_create(void** stream) {
    hipStream_t s;
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e == hipSuccess) *stream = s;
    return (int)e;
}

int llis_hip_stream_destroy(void* stream) { return (int)hipStreamDestroy(S(stream)); }
int llis_hip_stream_synchronize(void* stream) { return (int)hipStreamSynchronize(S(stream)); }

int llis_hip_stream_busy(void* stream) {
    hipError_t e = hipStreamQuery(S(stream));
    if (e == hipSuccess) return 0;
    if (e == hipErrorNotReady) return 1;
    return 1000 + (int)e;
}

int llis_hip_device_synchronize(void) { return (int)hipDeviceSynchronize(); }

int llis_hip_device_malloc(void** ptr, size_t bytes) { return (int)hipMalloc(ptr, bytes); }
int llis_hip_device_free(void* ptr) { return (int)hipFree(ptr); }

int llis_hip_host_alloc_coherent(void** ptr, size_t bytes) {
    return (int)hipHostMalloc(ptr, bytes, hipHostMallocCoherent | hipHostMallocMapped);
}

int llis_hip_host_alloc_pinned(void** ptr, size_t bytes) { return (int)hipHostMalloc(ptr, bytes, hipHostMallocDefault); }
int llis_hip_host_free(void* ptr) { return (int)hipHostFree(ptr); }

int llis_hip_memcpy(void* dst, const void* src, size_t bytes, int kind) { return (int)hipMemcpy(dst, src, bytes, kind_of(kind)); }

int llis_hip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, kind_of(kind), S(stream));
}

int llis_hip_fill_u32_async(void* dst, uint32_t value, size_t count, void* stream) {
    if (count == 0) return 0;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, S(stream),
                       reinterpret_cast<uint32_t*>(dst), value, count);
    return (int)hipGetLastError();
}

int llis_hip_launch_host_func(void* stream, void (*fn)(void*), void* arg) { return (int)hipLaunchHostFunc(S(stream), fn, arg); }

int llis_hip_launch_ring_marker(void* stream, uint64_t* slots, unsigned count, unsigned* cursor, uint64_t message) {
    if (!slots || !cursor || count == 0) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(ring_marker_kernel, dim3(1), dim3(1), 0, S(stream), slots, count - 1, cursor, message);
    return (int)hipGetLastError();
}

int llis_hip_event_create(void** event) {
    hipEvent_t ev;
    hipError_t e = hipEventCreate(&ev);
    if (e == hipSuccess) *event = ev;
    return (int)e;
}

int llis_hip_event_destroy(void* event) { return (int)hipEventDestroy(E(event)); }
int llis_hip_event_record(void* event, void* stream) { return (int)hipEventRecord(E(event), S(stream)); }
int llis_hip_event_synchronize(void* event) { return (int)hipEventSynchronize(E(event)); }
int llis_hip_event_elapsed_ms(void* start, void* stop, float* ms) { return (int)hipEventElapsedTime(ms, E(start), E(stop)); }

int llis_hip_profiler_start(void) { return (int)hipProfilerStart(); }
int llis_hip_profiler_stop(void) { return (int)hipProfilerStop(); }

}  // extern "C"
