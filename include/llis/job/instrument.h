#pragma once
// Un-aggregated workgroup hooks: every workgroup sends its own start and end message and stamps the
// compute unit it runs on.  The channel is passed by value as a kernel argument
// (reference include/llis/job/instrument.h:9-63, usage jobs/helloworld/helloworld.cu:8-29).

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/instrument_info.h>

namespace llis {
namespace job {

#if defined(__HIPCC__)

// Compute-unit id of the calling wave in 8 bits: XCC_ID << 5 | SE_ID << 3 | (CU_ID & 7).  Each of an XCD's four shader
// engines exposes eight consecutive CU_ID values (0..7 or 1..8 on MI355X), so the low three bits tell them apart and the
// id is dense over the 256 compute units, with the XCD in the top three bits.
__device__ __forceinline__ unsigned current_cu_id() {
    unsigned hw_id, xcc_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
    const unsigned cu = (hw_id >> 8) & 0xF;
    const unsigned se = (hw_id >> 13) & 0x7;
    return (((xcc_id & 0xF) << 5) | (se << 3) | (cu & 0x7)) & 0xFF;
}

__device__ __forceinline__ void kernel_start(JobId job_id, ipc::Gpu2SchedChannel* gpu2sched_channel) {
    if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
        InstrumentInfo info;
        info.is_start = 1;
        info.smid = (uint8_t)current_cu_id();
        info.num = 1;
        info.job_id = job_id;
        gpu2sched_channel->write(info);
    }
}

__device__ __forceinline__ void kernel_end(JobId job_id, ipc::Gpu2SchedChannel* gpu2sched_channel) {
    __syncthreads();
    if ((threadIdx.x | threadIdx.y | threadIdx.z) == 0) {
        InstrumentInfo info;
        info.is_start = 0;
        info.smid = (uint8_t)current_cu_id();
        info.num = 1;
        info.job_id = job_id;
        gpu2sched_channel->write(info);
    }
}

#endif  // __HIPCC__

}  // namespace job
}  // namespace llis
