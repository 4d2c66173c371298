#pragma once
// Result stores of the operator kernels.
//
// Each store is a relaxed device-scope atomic store, i.e. a write-through store (`global_store ... sc1`):
// the value goes past the XCD-private L2 to memory that all eight XCDs see, so a kernel that the
// scheduler launches on another stream right after this workgroup's end message finds it without any
// cache write-back in between (see FinishedBlockNotifier::end_written_through).

#include <hip/hip_runtime.h>

__device__ __forceinline__ void store_out(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ void store_out4(float* p, const float4& v) {
    store_out(p + 0, v.x);
    store_out(p + 1, v.y);
    store_out(p + 2, v.z);
    store_out(p + 3, v.w);
}
