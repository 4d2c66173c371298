// Memory-bound operators for gfx950 (fp32, NCHW, batch 1): dense (batch-1 GEMV), pooling, global average
// pool, fused elementwise, copy, softmax, LRN.  Each is bounded by HBM traffic, so the kernels aim at
// coalesced 16-byte accesses and wavefront (64-lane) reductions rather than at the matrix pipe.

#include <hip/hip_runtime.h>

#include <cfloat>
#include <cstring>

#include "paella_ops.h"
#include <llis/job/finished_block_notifier.h>

#include "launch.h"
#include "out_store.h"
#include "pool_body.h"
#include "dense_body.h"
#include "pack.h"

namespace {

using Notifier = llis::job::FinishedBlockNotifier;

__device__ __forceinline__ float act_apply(float v, int act, float slope, float lo, float hi) {
    switch (act) {
        case PAELLA_ACT_RELU:  return fmaxf(v, 0.f);
        case PAELLA_ACT_RELU6: return fminf(fmaxf(v, 0.f), 6.f);
        case PAELLA_ACT_PRELU: return v > 0.f ? v : v * slope;
        case PAELLA_ACT_CLIP:  return fminf(fmaxf(v, lo), hi);
        default:               return v;
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// ------------------------------------------------------------------------------------------ dense
// One wave per output row (dense_body.h).
__global__ __launch_bounds__(256) void dense_kernel(paella::DenseArgs a) {
    paella::hook_entry(a.notifier, a.job_id);
    paella::dense_row(a, (int)(blockIdx.x * 4 + (threadIdx.x >> 6)), (int)(threadIdx.x & 63));
    paella::hook_exit(a.notifier, a.job_id);
}

// Long rows (I >= kDenseLongRow, a multiple of 4): with one wave per row a layer of few, long rows (an embedding
// head: 512 rows of 100 KB) occupies half the SIMDs with one load in flight each.  Here a workgroup of eight
// waves owns two rows; each wave takes an eighth of both rows, keeps eight weight loads in flight per lane and
// uses every x value for both rows; the partial sums meet in LDS and are added in wave order (deterministic).
constexpr int kDenseLongRow = 8192;

__global__ __launch_bounds__(512) void dense_long_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         const float* __restrict__ bias, float* __restrict__ y, int I, int O,
                                                         int act, uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    __shared__ float part[2][8];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int o0 = blockIdx.x * 2;
    const int o1 = min(o0 + 1, O - 1);  // an odd O: the last workgroup reads its only row twice and stores it once
    const int I4 = I >> 2;
    const int per = (I4 + 7) >> 3;
    const int begin = wave * per;
    const int end = min(I4, begin + per);
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const float4* wa = reinterpret_cast<const float4*>(w + (size_t)o0 * I);
    const float4* wb = reinterpret_cast<const float4*>(w + (size_t)o1 * I);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f, b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
    auto dot = [](const float4& p, const float4& q) { return p.x * q.x + p.y * q.y + p.z * q.z + p.w * q.w; };
    int i = begin + lane;
    for (; i + 192 < end; i += 256) {
        const float4 p0 = wa[i], p1 = wa[i + 64], p2 = wa[i + 128], p3 = wa[i + 192];
        const float4 q0 = wb[i], q1 = wb[i + 64], q2 = wb[i + 128], q3 = wb[i + 192];
        const float4 v0 = x4[i], v1 = x4[i + 64], v2 = x4[i + 128], v3 = x4[i + 192];
        a0 += dot(p0, v0); a1 += dot(p1, v1); a2 += dot(p2, v2); a3 += dot(p3, v3);
        b0 += dot(q0, v0); b1 += dot(q1, v1); b2 += dot(q2, v2); b3 += dot(q3, v3);
    }
    for (; i < end; i += 64) {
        const float4 v = x4[i];
        a0 += dot(wa[i], v);
        b0 += dot(wb[i], v);
    }
    const float sa = wave_sum((a0 + a1) + (a2 + a3));
    const float sb = wave_sum((b0 + b1) + (b2 + b3));
    if (lane == 0) {
        part[0][wave] = sa;
        part[1][wave] = sb;
    }
    __syncthreads();
    if (threadIdx.x < 2) {
        const int o = o0 + (int)threadIdx.x;
        if (o < O) {
            float v = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) v += part[threadIdx.x][k];
            store_out(y + o, act_apply(v + (bias ? bias[o] : 0.f), act, 0.f, 0.f, 0.f));
        }
    }
    paella::hook_exit(notifier, job_id);
}

// ------------------------------------------------------------------------------------------ pooling
using paella::PoolArgs;

__global__ __launch_bounds__(256) void pool_kernel(PoolArgs p) {
    paella::hook_entry(p.notifier, p.job_id);
    paella::pool_element(p, (int)(blockIdx.x * 256 + threadIdx.x));
    paella::hook_exit(p.notifier, p.job_id);
}

// One wave per channel.
__global__ __launch_bounds__(256) void gap_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int HW,
                                                  uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c < C) {
        const float* xc = x + (size_t)c * HW;
        float acc = 0.f;
        for (int i = lane; i < HW; i += 64) acc += xc[i];
        acc = wave_sum(acc);
        if (lane == 0) store_out(y + c, acc / (float)HW);
    }
    paella::hook_exit(notifier, job_id);
}

// ------------------------------------------------------------------------------------------ elementwise
struct EltArgs {
    const float* a;
    const float* b;
    const float* scale;
    const float* shift;
    const float* slope;
    float* y;
    int C, HW;
    int act;
    float lo, hi;
    uint32_t job_id;
    Notifier* notifier;
};

__device__ __forceinline__ float elt_one(const EltArgs& p, float a, float b, int c) {
    float v = a;
    if (p.scale) v *= p.scale[c];
    if (p.shift) v += p.shift[c];
    v += b;
    return act_apply(v, p.act, p.act == PAELLA_ACT_PRELU ? p.slope[c] : 0.f, p.lo, p.hi);
}

template <bool VEC4>
__global__ __launch_bounds__(256) void eltwise_kernel(EltArgs p) {
    paella::hook_entry(p.notifier, p.job_id);
    const size_t n = (size_t)p.C * p.HW;
    if (VEC4) {
        const size_t i4 = (size_t)blockIdx.x * 256 + threadIdx.x;
        if (i4 * 4 < n) {
            const int c = (int)((i4 * 4) / p.HW);  // HW % 4 == 0: the four lanes share a channel
            const float4 a = reinterpret_cast<const float4*>(p.a)[i4];
            float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p.b) b = reinterpret_cast<const float4*>(p.b)[i4];
            float4 r;
            r.x = elt_one(p, a.x, b.x, c);
            r.y = elt_one(p, a.y, b.y, c);
            r.z = elt_one(p, a.z, b.z, c);
            r.w = elt_one(p, a.w, b.w, c);
            store_out4(p.y, i4 * 4, r);
        }
    } else {
        const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
        if (i < n) store_out(p.y + i, elt_one(p, p.a[i], p.b ? p.b[i] : 0.f, (int)(i / p.HW)));
    }
    paella::hook_exit(p.notifier, p.job_id);
}

__global__ __launch_bounds__(256) void copy_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n,
                                                   uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n && n < ((size_t)1 << 30) && ((((uintptr_t)x | (uintptr_t)y) & 15) == 0)) {
        store_out4(y, i, *reinterpret_cast<const float4*>(x + i));
    } else {
        for (size_t k = i; k < n && k < i + 4; ++k) store_out(y + k, x[k]);
    }
    paella::hook_exit(notifier, job_id);
}

// ------------------------------------------------------------------------------------------ softmax / LRN
// One workgroup per row.
__global__ __launch_bounds__(256) void softmax_kernel(const float* __restrict__ x, float* __restrict__ y, int cols,
                                                      uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    __shared__ float part[4];
    const float* xr = x + (size_t)blockIdx.x * cols;
    float* yr = y + (size_t)blockIdx.x * cols;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float m = -FLT_MAX;
    for (int i = threadIdx.x; i < cols; i += 256) m = fmaxf(m, xr[i]);
    m = wave_max(m);
    if (lane == 0) part[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    __syncthreads();
    float s = 0.f;
    for (int i = threadIdx.x; i < cols; i += 256) s += expf(xr[i] - m);
    s = wave_sum(s);
    if (lane == 0) part[wave] = s;
    __syncthreads();
    s = (part[0] + part[1]) + (part[2] + part[3]);
    for (int i = threadIdx.x; i < cols; i += 256) store_out(yr + i, expf(xr[i] - m) / s);
    paella::hook_exit(notifier, job_id);
}

// Rows of at most kSoftmaxShortRow values (the face detector's two class scores per anchor box: 4420 rows of 2): one thread
// per row instead of a workgroup of 256 for a handful of values.  The row's sum runs left to right.
constexpr int kSoftmaxShortRow = 8;

__global__ __launch_bounds__(256) void softmax_short_kernel(const float* __restrict__ x, float* __restrict__ y, int rows, int cols,
                                                            uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r < rows) {
        float v[kSoftmaxShortRow];
        float m = -FLT_MAX;
#pragma unroll
        for (int i = 0; i < kSoftmaxShortRow; ++i) {
            v[i] = i < cols ? x[(size_t)r * cols + i] : -FLT_MAX;
            m = fmaxf(m, v[i]);
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kSoftmaxShortRow; ++i) {
            v[i] = i < cols ? expf(v[i] - m) : 0.f;
            s += v[i];
        }
#pragma unroll
        for (int i = 0; i < kSoftmaxShortRow; ++i)
            if (i < cols) store_out(y + (size_t)r * cols + i, v[i] / s);
    }
    paella::hook_exit(notifier, job_id);
}

__global__ __launch_bounds__(256) void lrn_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int HW, int size,
                                                  float alpha, float beta, float k, uint32_t job_id, Notifier* notifier) {
    paella::hook_entry(notifier, job_id);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx < (size_t)C * HW) {
        const int c = (int)(idx / HW);
        const int i = (int)(idx - (size_t)c * HW);
        const int lo = (size - 1) / 2, hi = size - 1 - lo;
        float sq = 0.f;
        if (size == 5) {
            // the window the served models use: its five loads leave together (a channel outside the tensor reads the
            // centre instead and counts as zero); same sum in the same order as the loop below
            float v[5];
#pragma unroll
            for (int t = 0; t < 5; ++t) {
                const int cc = c - 2 + t;
                const bool ok = cc >= 0 && cc < C;
                const float u = x[(size_t)(ok ? cc : c) * HW + i];
                v[t] = ok ? u : 0.f;
            }
#pragma unroll
            for (int t = 0; t < 5; ++t) sq += v[t] * v[t];
            store_out(y + idx, v[2] / powf(k + alpha / (float)size * sq, beta));
        } else {
            for (int cc = max(0, c - lo); cc <= min(C - 1, c + hi); ++cc) {
                const float v = x[(size_t)cc * HW + i];
                sq += v * v;
            }
            store_out(y + idx, x[idx] / powf(k + alpha / (float)size * sq, beta));
        }
    }
    paella::hook_exit(notifier, job_id);
}

inline unsigned blocks_for(size_t n, unsigned per_block) { return (unsigned)((n + per_block - 1) / per_block); }

inline void set_dims(paella_launch_dims* d, unsigned grid, unsigned block, unsigned lds, unsigned vgprs) {
    d->grid = grid;
    d->block = block;
    d->lds_bytes = lds;
    d->vgprs = vgprs;
}

}  // namespace

paella::TimingEvents& paella::timing_events() {
    static thread_local paella::TimingEvents events;
    return events;
}

extern "C" {

int paella_pool_out(int in, int k, int stride, int pad, int ceil_mode) {
    const int num = in + 2 * pad - k;
    int out;
    if (ceil_mode) {
        out = (num + stride - 1) / stride + 1;
        if ((out - 1) * stride >= in + pad) --out;  // the last window must start inside input + left padding
    } else {
        out = num / stride + 1;
    }
    return out;
}

static bool dense_long(int I) { return I >= kDenseLongRow && (I & 3) == 0; }

int paella_dense_dims(int I, int O, paella_launch_dims* dims) {
    if (I <= 0 || O <= 0 || !dims) return PAELLA_EINVAL;
    if (dense_long(I)) set_dims(dims, blocks_for(O, 2), 512, 64, 48);
    else set_dims(dims, blocks_for(O, 4), 256, 0, 32);
    return 0;
}

int paella_dense_launch(const float* x, const float* w, const float* bias, float* y, int I, int O, int act, void* stream,
                        uint32_t job_id, void* notifier) {
    if (!x || !w || !y || I <= 0 || O <= 0 || act < 0 || act > PAELLA_ACT_RELU6) return PAELLA_EINVAL;
    if (dense_long(I))
        paella::launch(dense_long_kernel, dim3(blocks_for(O, 2)), dim3(512), 0, (hipStream_t)stream, x, w, bias, y, I, O, act, job_id,
                       (Notifier*)notifier);
    else {
        paella::DenseArgs a{x, w, bias, y, I, O, act, job_id, 0u, (Notifier*)notifier};
        if (paella::pack_record_dense(a, stream)) return 0;
        paella::launch(dense_kernel, dim3(blocks_for(O, 4)), dim3(256), 0, (hipStream_t)stream, a);
    }
    return (int)hipGetLastError();
}

static int pool_check(const paella_pool_desc* d, int* P, int* Q) {
    if (!d || d->C <= 0 || d->H <= 0 || d->W <= 0 || d->R <= 0 || d->S <= 0 || d->stride_h <= 0 || d->stride_w <= 0 ||
        d->pad_h < 0 || d->pad_w < 0 || d->pad_h * 2 > d->R || d->pad_w * 2 > d->S)
        return PAELLA_EINVAL;
    *P = paella_pool_out(d->H, d->R, d->stride_h, d->pad_h, d->ceil_mode);
    *Q = paella_pool_out(d->W, d->S, d->stride_w, d->pad_w, d->ceil_mode);
    return (*P > 0 && *Q > 0) ? 0 : PAELLA_EINVAL;
}

int paella_pool2d_dims(const paella_pool_desc* d, paella_launch_dims* dims) {
    int P, Q;
    if (int rc = pool_check(d, &P, &Q)) return rc;
    if (!dims) return PAELLA_EINVAL;
    set_dims(dims, blocks_for((size_t)d->C * P * Q, 256), 256, 0, 32);
    return 0;
}

int paella_pool2d_launch(const paella_pool_desc* d, const float* x, float* y, void* stream, uint32_t job_id, void* notifier) {
    PoolArgs a;
    if (!x || !y || !paella::pool_fill_args(d, x, y, job_id, notifier, &a)) return PAELLA_EINVAL;
    const int P = a.P, Q = a.Q;
    if (paella::pack_record_pool(a, stream)) return 0;
    paella::launch(pool_kernel, dim3(blocks_for((size_t)d->C * P * Q, 256)), dim3(256), 0, (hipStream_t)stream, a);
    return (int)hipGetLastError();
}

int paella_global_avgpool_dims(int C, int HW, paella_launch_dims* dims) {
    if (C <= 0 || HW <= 0 || !dims) return PAELLA_EINVAL;
    set_dims(dims, blocks_for(C, 4), 256, 0, 32);
    return 0;
}

int paella_global_avgpool_launch(const float* x, float* y, int C, int HW, void* stream, uint32_t job_id, void* notifier) {
    if (!x || !y || C <= 0 || HW <= 0) return PAELLA_EINVAL;
    paella::launch(gap_kernel, dim3(blocks_for(C, 4)), dim3(256), 0, (hipStream_t)stream, x, y, C, HW, job_id, (Notifier*)notifier);
    return (int)hipGetLastError();
}

int paella_eltwise_dims(int C, int HW, paella_launch_dims* dims) {
    if (C <= 0 || HW <= 0 || !dims) return PAELLA_EINVAL;
    const size_t n = (size_t)C * HW;
    set_dims(dims, (HW & 3) == 0 ? blocks_for(n / 4, 256) : blocks_for(n, 256), 256, 0, 32);
    return 0;
}

int paella_eltwise_launch(const float* a, const float* b, const float* scale, const float* shift, const float* slope, float* y,
                          int C, int HW, int act, float lo, float hi, void* stream, uint32_t job_id, void* notifier) {
    if (!a || !y || C <= 0 || HW <= 0 || act < 0 || act > PAELLA_ACT_CLIP) return PAELLA_EINVAL;
    if (act == PAELLA_ACT_PRELU && !slope) return PAELLA_EINVAL;
    EltArgs p;
    p.a = a; p.b = b; p.scale = scale; p.shift = shift; p.slope = slope; p.y = y;
    p.C = C; p.HW = HW; p.act = act; p.lo = lo; p.hi = hi;
    p.job_id = job_id; p.notifier = (Notifier*)notifier;
    const size_t n = (size_t)C * HW;
    const bool aligned = ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15) == 0);
    if ((HW & 3) == 0 && aligned && n < ((size_t)1 << 30)) {
        paella::launch(eltwise_kernel<true>, dim3(blocks_for(n / 4, 256)), dim3(256), 0, (hipStream_t)stream, p);
    } else {
        paella::launch(eltwise_kernel<false>, dim3(blocks_for(n, 256)), dim3(256), 0, (hipStream_t)stream, p);
    }
    return (int)hipGetLastError();
}

int paella_copy_dims(size_t n, paella_launch_dims* dims) {
    if (n == 0 || !dims) return PAELLA_EINVAL;
    set_dims(dims, blocks_for((n + 3) / 4, 256), 256, 0, 16);
    return 0;
}

int paella_copy_launch(const float* x, float* y, size_t n, void* stream, uint32_t job_id, void* notifier) {
    if (!x || !y || n == 0) return PAELLA_EINVAL;
    paella::launch(copy_kernel, dim3(blocks_for((n + 3) / 4, 256)), dim3(256), 0, (hipStream_t)stream, x, y, n, job_id,
                       (Notifier*)notifier);
    return (int)hipGetLastError();
}

int paella_softmax_dims(int rows, int cols, paella_launch_dims* dims) {
    if (rows <= 0 || cols <= 0 || !dims) return PAELLA_EINVAL;
    if (cols <= kSoftmaxShortRow) set_dims(dims, blocks_for((size_t)rows, 256), 256, 0, 32);
    else set_dims(dims, (unsigned)rows, 256, 16, 32);
    return 0;
}

int paella_softmax_launch(const float* x, float* y, int rows, int cols, void* stream, uint32_t job_id, void* notifier) {
    if (!x || !y || rows <= 0 || cols <= 0) return PAELLA_EINVAL;
    if (cols <= kSoftmaxShortRow)
        paella::launch(softmax_short_kernel, dim3(blocks_for((size_t)rows, 256)), dim3(256), 0, (hipStream_t)stream, x, y, rows, cols, job_id,
                       (Notifier*)notifier);
    else
        paella::launch(softmax_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, x, y, cols, job_id, (Notifier*)notifier);
    return (int)hipGetLastError();
}

int paella_lrn_dims(int C, int HW, paella_launch_dims* dims) {
    if (C <= 0 || HW <= 0 || !dims) return PAELLA_EINVAL;
    set_dims(dims, blocks_for((size_t)C * HW, 256), 256, 0, 32);
    return 0;
}

int paella_lrn_launch(const float* x, float* y, int C, int HW, int size, float alpha, float beta, float k, void* stream,
                      uint32_t job_id, void* notifier) {
    if (!x || !y || C <= 0 || HW <= 0 || size <= 0) return PAELLA_EINVAL;
    paella::launch(lrn_kernel, dim3(blocks_for((size_t)C * HW, 256)), dim3(256), 0, (hipStream_t)stream, x, y, C, HW, size, alpha,
                       beta, k, job_id, (Notifier*)notifier);
    return (int)hipGetLastError();
}

int paella_ops_time_launches(void* start_event, void* stop_event) {
    if ((start_event == nullptr) != (stop_event == nullptr)) return PAELLA_EINVAL;
    paella::TimingEvents& t = paella::timing_events();
    t.start = (hipEvent_t)start_event;
    t.stop = (hipEvent_t)stop_event;
    return 0;
}

static const void* family_kernel(const char* family) {
    if (!std::strcmp(family, "dense")) return (const void*)dense_kernel;
    if (!std::strcmp(family, "dense_long")) return (const void*)dense_long_kernel;
    if (!std::strcmp(family, "pool")) return (const void*)pool_kernel;
    if (!std::strcmp(family, "gap")) return (const void*)gap_kernel;
    if (!std::strcmp(family, "eltwise")) return (const void*)eltwise_kernel<true>;
    if (!std::strcmp(family, "copy")) return (const void*)copy_kernel;
    if (!std::strcmp(family, "softmax")) return (const void*)softmax_kernel;
    if (!std::strcmp(family, "softmax_short")) return (const void*)softmax_short_kernel;
    if (!std::strcmp(family, "lrn")) return (const void*)lrn_kernel;
    return nullptr;
}

int paella_kernel_occupancy(const char* family, unsigned block, unsigned lds_bytes, int* blocks_per_cu) {
    if (!family || !blocks_per_cu || block == 0) return PAELLA_EINVAL;
    const void* fn = family_kernel(family);
    if (!fn) return PAELLA_EINVAL;
    return (int)hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, fn, (int)block, lds_bytes);
}

int paella_kernel_static_lds(const char* family, unsigned* lds_bytes) {
    if (!family || !lds_bytes) return PAELLA_EINVAL;
    const void* fn = family_kernel(family);
    if (!fn) return PAELLA_EINVAL;
    hipFuncAttributes attr;
    hipError_t e = hipFuncGetAttributes(&attr, fn);
    if (e != hipSuccess) return (int)e;
    *lds_bytes = (unsigned)attr.sharedSizeBytes;
    return 0;
}

int paella_kernel_vgprs(const char* family, unsigned* vgprs) {
    if (!family || !vgprs) return PAELLA_EINVAL;
    const void* fn = family_kernel(family);
    if (!fn) return PAELLA_EINVAL;
    hipFuncAttributes attr;
    hipError_t e = hipFuncGetAttributes(&attr, fn);
    if (e != hipSuccess) return (int)e;
    *vgprs = (unsigned)attr.numRegs;
    return 0;
}

}  // extern "C"
