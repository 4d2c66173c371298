#pragma once
// Dense layer for rows below the long-row limit, one wave per output row; shared by the dense kernel and by the conv
// group kernel when a launch carries the dense layers of several requests.

#include <hip/hip_runtime.h>

#include "paella_ops.h"
#include <llis/job/finished_block_notifier.h>

#include "out_store.h"

namespace paella {

struct DenseArgs {
    const float* x;
    const float* w;     // [O][I]
    const float* bias;  // may be null
    float* y;
    int I, O, act;
    uint32_t job_id;
    unsigned hook_blocks;  // workgroups of the launch that report to `notifier`; 0: all of them (one job per launch)
    llis::job::FinishedBlockNotifier* notifier;
};

__device__ __forceinline__ float dense_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Output row o by the calling wave (all 64 lanes take part; nothing happens for o >= O).  Lanes stride the row with
// float4 loads (x stays in L1/L2).
__device__ __forceinline__ void dense_row(const DenseArgs& a, const int o, const int lane) {
    if (o >= a.O) return;
    const int I = a.I;
    const float* __restrict__ x = a.x;
    const float* __restrict__ wr = a.w + (size_t)o * I;
    float acc = 0.f;
    if ((I & 3) == 0) {
        const float4* w4 = reinterpret_cast<const float4*>(wr);
        const float4* x4 = reinterpret_cast<const float4*>(x);
        // four independent loads and sums per trip: a row of 2048 floats is two trips to memory, not eight
        const int I4 = I / 4;
        float a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int i = lane;
        for (; i + 192 < I4; i += 256) {
            const float4 p0 = w4[i], p1 = w4[i + 64], p2 = w4[i + 128], p3 = w4[i + 192];
            const float4 q0 = x4[i], q1 = x4[i + 64], q2 = x4[i + 128], q3 = x4[i + 192];
            acc += p0.x * q0.x + p0.y * q0.y + p0.z * q0.z + p0.w * q0.w;
            a1 += p1.x * q1.x + p1.y * q1.y + p1.z * q1.z + p1.w * q1.w;
            a2 += p2.x * q2.x + p2.y * q2.y + p2.z * q2.z + p2.w * q2.w;
            a3 += p3.x * q3.x + p3.y * q3.y + p3.z * q3.z + p3.w * q3.w;
        }
        for (; i < I4; i += 64) {
            const float4 p = w4[i], q = x4[i];
            acc += p.x * q.x + p.y * q.y + p.z * q.z + p.w * q.w;
        }
        acc = (acc + a1) + (a2 + a3);
    } else {
        for (int i = lane; i < I; i += 64) acc += wr[i] * x[i];
    }
    acc = dense_wave_sum(acc);
    if (lane == 0) {
        float v = acc + (a.bias ? a.bias[o] : 0.f);
        if (a.act == PAELLA_ACT_RELU) v = fmaxf(v, 0.f);
        else if (a.act == PAELLA_ACT_RELU6) v = fminf(fmaxf(v, 0.f), 6.f);
        store_out(a.y + o, v);
    }
}

}  // namespace paella
