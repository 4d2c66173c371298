#pragma once
// Result stores of the operator kernels.
//
// Each store is a relaxed device-scope atomic store, i.e. a write-through store (`global_store ... sc1`):
// the value goes past the XCD-private L2 to memory that all eight XCDs see, so a kernel that the
// scheduler launches on another stream right after this workgroup's end message finds it without any
// cache write-back in between (see FinishedBlockNotifier::end_written_through).

#include <hip/hip_runtime.h>

#include "paella_ops.h"
#include <llis/job/finished_block_notifier.h>

namespace paella {
// First statement of every operator kernel.  The start message is sent only when the scheduler asked for it
// (job id without PAELLA_JOB_ID_NO_START); the entry clock sample for per-workgroup timing is taken when start()
// runs (it knows from the notifier) or when the caller set PAELLA_JOB_ID_TIME_BLOCKS.
__device__ __forceinline__ void hook_entry(llis::job::FinishedBlockNotifier* notifier, uint32_t job_id) {
    if (notifier) {
        if (!(job_id & PAELLA_JOB_ID_NO_START)) notifier->start(job_id & ~PAELLA_JOB_ID_FLAGS);
        else if (job_id & PAELLA_JOB_ID_TIME_BLOCKS) notifier->begin_timing();
    }
}

// The same for a workgroup of a launch that carries several jobs' kernels: `blocks` workgroups report to this notifier.
__device__ __forceinline__ void hook_entry(llis::job::FinishedBlockNotifier* notifier, uint32_t job_id, unsigned blocks) {
    if (notifier) {
        if (!(job_id & PAELLA_JOB_ID_NO_START)) notifier->start(job_id & ~PAELLA_JOB_ID_FLAGS, blocks);
        else if (job_id & PAELLA_JOB_ID_TIME_BLOCKS) notifier->begin_timing();
    }
}

// Last statement of every operator kernel (all results written with store_out / store_out4).
__device__ __forceinline__ void hook_exit(llis::job::FinishedBlockNotifier* notifier, uint32_t job_id) {
    if (notifier) notifier->end_written_through(job_id & ~PAELLA_JOB_ID_FLAGS, (job_id & PAELLA_JOB_ID_TIME_BLOCKS) != 0);
}
__device__ __forceinline__ void hook_exit(llis::job::FinishedBlockNotifier* notifier, uint32_t job_id, unsigned blocks) {
    if (notifier) notifier->end_written_through(job_id & ~PAELLA_JOB_ID_FLAGS, (job_id & PAELLA_JOB_ID_TIME_BLOCKS) != 0, blocks);
}
}  // namespace paella

__device__ __forceinline__ void store_out(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Four consecutive floats at base[index .. index+3] (16-byte aligned) as ONE 16-byte write-through store.  Four
// separate dword stores per lane would be 16 bytes apart across lanes: sixteen partial-line writes per
// instruction instead of full lines.  `base` must be uniform over the wave; index * 4 must fit 32 bits.
__device__ __forceinline__ void store_out4(float* base, size_t index, const float4& v) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xFFFFFFFFu, 0x00027000);
    const u32x4 bits = {__builtin_bit_cast(unsigned, v.x), __builtin_bit_cast(unsigned, v.y), __builtin_bit_cast(unsigned, v.z),
                        __builtin_bit_cast(unsigned, v.w)};
    __builtin_amdgcn_raw_buffer_store_b128(bits, rsrc, (int)(unsigned)(index * 4), 0, 16 /* sc1: write through */);
}
