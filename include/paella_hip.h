/*
 * paella_hip.h -- thin C-ABI over the HIP runtime used by the llis server, job adapters and benches.
 *
 * Every place where the reference calls the CUDA runtime directly goes through one of these functions
 * instead, so the host-side C++ (scheduler, channels, RegisteredJob) carries no HIP types and can be
 * linked against a scripted test double on machines without a GPU.  Return value: 0 on success, else the
 * hipError_t value; llis_hip_error_string() names it.  Handles are opaque void*.
 *
 * Reference call sites replaced (all paths relative to the reference tree):
 *   stream pool               cudaStreamCreate            src/server/scheduler_full3.cpp:42-44
 *   mem-stage completion      cudaLaunchHostFunc          src/server/scheduler_full3.cpp:429-431
 *   ring allocation           cudaHostRegister/cudaMalloc src/ipc/shm_primitive_channel.cu:107-124
 *   notifier array            cudaMalloc/cudaMemcpy       src/job/finished_block_notifier.cu:27-39
 *   I/O pool pinning          cudaHostRegister            src/server/registered_job.cpp:102
 *   occupancy budget          cudaGetDeviceProperties     src/server/sm_resources.cpp:17-24
 *   profiler toggles          cudaProfilerStart/Stop      src/server/server.cpp:64-70
 *   per-request copies        cudaMemcpyAsync             jobs/tvm_mnist/tvm_mnist.cpp:38,46
 */
#ifndef PAELLA_HIP_H
#define PAELLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum llis_hip_copy_kind { LLIS_HIP_H2D = 1, LLIS_HIP_D2H = 2, LLIS_HIP_D2D = 3 };

/* Aggregate occupancy budget of the device, in the units SmResources accounts in. */
typedef struct llis_hip_device_caps {
    int num_cus;                  /* compute units (256 on MI355X) */
    int wavefront_size;           /* 64 */
    int max_threads_per_cu;       /* resident threads per CU */
    int max_blocks_per_cu;        /* resident workgroups per CU: one per wave slot (32) */
    int vgprs_per_cu;             /* vector-register lanes per CU: 4 SIMDs x 512 registers x 64 lanes (131072) */
    int lds_bytes_per_cu;         /* 160 KiB on gfx950 */
    int clock_khz;
    int l2_bytes;
    char name[64];
} llis_hip_device_caps;

int llis_hip_device_count(int* count);
int llis_hip_set_device(int device);
int llis_hip_get_device_caps(llis_hip_device_caps* caps);
const char* llis_hip_error_string(int code);

int llis_hip_stream_create(void** stream);
int llis_hip_stream_destroy(void* stream);
int llis_hip_stream_synchronize(void* stream);
/* 0 = idle, 1 = still busy, <0 never; other positive values are errors shifted by 1000 */
int llis_hip_stream_busy(void* stream);
int llis_hip_device_synchronize(void);

int llis_hip_device_malloc(void** ptr, size_t bytes);
int llis_hip_device_free(void* ptr);
/* Fine-grained, device-mapped, system-coherent host memory: the notification ring lives here. */
int llis_hip_host_alloc_coherent(void** ptr, size_t bytes);
/* Ordinary pinned host memory for request staging buffers. */
int llis_hip_host_alloc_pinned(void** ptr, size_t bytes);
int llis_hip_host_free(void* ptr);

int llis_hip_memcpy(void* dst, const void* src, size_t bytes, int kind);
int llis_hip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);
/* Fill kernel (not a memset node), safe to capture into graphs. */
int llis_hip_fill_u32_async(void* dst, uint32_t value, size_t count, void* stream);

/* Runs fn(arg) on a runtime thread once all prior work on the stream has finished. */
int llis_hip_launch_host_func(void* stream, void (*fn)(void*), void* arg);

/*
 * Enqueues a one-lane kernel that publishes `message` (a 64-bit ring slot value) into the notification
 * ring {slots, count, cursor} once all prior work on the stream has finished.  This is how a memory-copy
 * stage reports completion without a host callback thread.
 */
int llis_hip_launch_ring_marker(void* stream, uint64_t* slots, unsigned count, unsigned* cursor, uint64_t message);

int llis_hip_event_create(void** event);
int llis_hip_event_destroy(void* event);
int llis_hip_event_record(void* event, void* stream);
int llis_hip_event_synchronize(void* event);
int llis_hip_event_elapsed_ms(void* start, void* stop, float* ms);

int llis_hip_profiler_start(void);
int llis_hip_profiler_stop(void);

#ifdef __cplusplus
}
#endif
#endif
