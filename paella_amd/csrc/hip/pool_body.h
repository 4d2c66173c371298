#pragma once
// Pooling, one thread per output element; shared by the pooling kernel and by the conv group kernel that carries a
// pooling operator along (the branches of an inception module start with three 1x1 convs and a pool that all read the
// module's input).

#include <hip/hip_runtime.h>

#include <cfloat>

#include "paella_ops.h"
#include <llis/job/finished_block_notifier.h>

#include "out_store.h"

namespace paella {

struct PoolArgs {
    const float* x;
    float* y;
    int C, H, W, P, Q, R, S, sh, sw, ph, pw;
    int is_avg, count_include_pad;
    uint32_t job_id;
    unsigned hook_blocks;  // workgroups of the launch that report to `notifier`; 0: all of them (one job per launch)
    llis::job::FinishedBlockNotifier* notifier;
    // 3 x 3 and 2 x 2 windows whose sizes the host has checked (fast = 1): output column and row by multiply-high
    // (floor(a / d) = umulhi(a, mul) + (a & one), exact while a * d < 2^32), operands through buffer descriptors with 32-bit offsets
    unsigned div_q_mul, div_q_one, div_p_mul, div_p_one;
    int fast;
    unsigned x_bytes, out_bytes;
};

// One window with its size known at compile time: every load of the window leaves before the first result is needed (a tap
// outside the image reads element 0 of the channel and is ignored afterwards).  Same operations in the same order as the
// generic loop, so the same bits.
template <int R, int S>
__device__ __forceinline__ float pool_window(const PoolArgs& p, const float* xc, int h0, int w0) {
    float v[R * S];
    bool ok[R * S];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int h = h0 + r, w = w0 + s;
            ok[r * S + s] = (unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W;
            v[r * S + s] = xc[ok[r * S + s] ? h * p.W + w : 0];
        }
    if (p.is_avg) {
        float acc = 0.f;
        int valid = 0;
#pragma unroll
        for (int t = 0; t < R * S; ++t)
            if (ok[t]) {
                acc += v[t];
                ++valid;
            }
        int div = valid;
        if (p.count_include_pad) {
            const int he = min(h0 + R, p.H + p.ph), we = min(w0 + S, p.W + p.pw);
            div = (he - h0) * (we - w0);
        }
        return div ? acc / (float)div : 0.f;
    }
    float m = -FLT_MAX;
#pragma unroll
    for (int t = 0; t < R * S; ++t)
        if (ok[t]) m = fmaxf(m, v[t]);
    return m;
}

// The same window with 32-bit offsets into buffer descriptors and without a branch per tap.  A pooling operator that shares a
// launch with convs runs on the compute units their waves run on, and a vector instruction takes matrix-pipe time there: the
// plain form above spends some 190 vector instructions per element, most of them on 64-bit addresses, two divisions and
// per-tap bounds.  Average: a tap outside the image gets an offset beyond any length and reads as the zero it adds (the sum
// starts at +0, so an added zero changes no bit), and the number of valid taps is valid rows times valid columns.  Maximum:
// rows and columns are clamped into the image, which re-reads elements of the same window (pad <= size / 2: a window always
// holds an element of the image), and a maximum does not change with repeated operands.  A thread past the last element works
// on the last one and has its store dropped.
template <int R, int S>
__device__ __forceinline__ void pool_window_fast(const PoolArgs& p, const int idx) {
    const int total = p.C * p.P * p.Q;
    const bool live = idx < total;
    const int e = live ? idx : total - 1;
    // every factor below is under 2^23 (checked by the host): 24-bit multiplies
    const int row = (int)(__umulhi((unsigned)e, p.div_q_mul) + ((unsigned)e & p.div_q_one));  // over (channel, output row)
    const int qo = e - __mul24(row, p.Q);
    const int c = (int)(__umulhi((unsigned)row, p.div_p_mul) + ((unsigned)row & p.div_p_one));
    const int po = row - __mul24(c, p.P);
    const int h0 = __mul24(po, p.sh) - p.ph, w0 = __mul24(qo, p.sw) - p.pw;
    const int crow = __mul24(c, p.H);
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)p.x, 0, p.x_bytes, 0x00027000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc((void*)p.y, 0, p.out_bytes, 0x00027000);
    float v[R * S];
    float result;
    if (p.is_avg) {
        constexpr int kBad = 0x40000000;  // one of them, or two added, is past any length (x_bytes < 2^30)
        int row_off[R], col_off[S];
#pragma unroll
        for (int r = 0; r < R; ++r) row_off[r] = (unsigned)(h0 + r) < (unsigned)p.H ? __mul24(crow + h0 + r, p.W) * 4 : kBad;
#pragma unroll
        for (int t = 0; t < S; ++t) col_off[t] = (unsigned)(w0 + t) < (unsigned)p.W ? (w0 + t) * 4 : kBad;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < S; ++t) v[r * S + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, row_off[r] + col_off[t], 0, 0));
        float acc = 0.f;
#pragma unroll
        for (int t = 0; t < R * S; ++t) acc += v[t];
        int div;
        if (p.count_include_pad) {
            const int he = min(h0 + R, p.H + p.ph), we = min(w0 + S, p.W + p.pw);
            div = (he - h0) * (we - w0);
        } else {
            div = (min(h0 + R, p.H) - max(h0, 0)) * (min(w0 + S, p.W) - max(w0, 0));
        }
        result = div ? acc / (float)div : 0.f;
    } else {
        int row_off[R], col_off[S];
#pragma unroll
        for (int r = 0; r < R; ++r) row_off[r] = __mul24(crow + min(max(h0 + r, 0), p.H - 1), p.W) * 4;
#pragma unroll
        for (int t = 0; t < S; ++t) col_off[t] = min(max(w0 + t, 0), p.W - 1) * 4;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < S; ++t) v[r * S + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, row_off[r] + col_off[t], 0, 0));
        float m = -FLT_MAX;
#pragma unroll
        for (int t = 0; t < R * S; ++t) m = fmaxf(m, v[t]);
        result = m;
    }
    // write-through (sc1), like store_out
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, result), yr, live ? e * 4 : -1, 0, 16);
}

// Output element number idx (channel-major, then row, then column); does nothing past the last element.
__device__ __forceinline__ void pool_element(const PoolArgs& p, const int idx) {
    if (p.fast) {
        if (p.R == 3) pool_window_fast<3, 3>(p, idx);
        else pool_window_fast<2, 2>(p, idx);
        return;
    }
    const int PQ = p.P * p.Q;
    if (idx < p.C * PQ) {
        const int c = idx / PQ;
        const int pix = idx - c * PQ;
        const int po = pix / p.Q;
        const int qo = pix - po * p.Q;
        const float* xc = p.x + (size_t)c * p.H * p.W;
        const int h0 = po * p.sh - p.ph, w0 = qo * p.sw - p.pw;
        if (p.R == 3 && p.S == 3) {
            store_out(p.y + idx, pool_window<3, 3>(p, xc, h0, w0));
        } else if (p.R == 2 && p.S == 2) {
            store_out(p.y + idx, pool_window<2, 2>(p, xc, h0, w0));
        } else if (p.is_avg) {
            float acc = 0.f;
            int valid = 0;
            for (int r = 0; r < p.R; ++r) {
                const int h = h0 + r;
                if ((unsigned)h >= (unsigned)p.H) continue;
                for (int s = 0; s < p.S; ++s) {
                    const int w = w0 + s;
                    if ((unsigned)w >= (unsigned)p.W) continue;
                    acc += xc[(size_t)h * p.W + w];
                    ++valid;
                }
            }
            int div = valid;
            if (p.count_include_pad) {
                // window clipped to the padded extent [-pad, in + pad)
                const int he = min(h0 + p.R, p.H + p.ph), we = min(w0 + p.S, p.W + p.pw);
                div = (he - h0) * (we - w0);
            }
            store_out(p.y + idx, div ? acc / (float)div : 0.f);
        } else {
            float m = -FLT_MAX;
            for (int r = 0; r < p.R; ++r) {
                const int h = h0 + r;
                if ((unsigned)h >= (unsigned)p.H) continue;
                for (int s = 0; s < p.S; ++s) {
                    const int w = w0 + s;
                    if ((unsigned)w >= (unsigned)p.W) continue;
                    m = fmaxf(m, xc[(size_t)h * p.W + w]);
                }
            }
            store_out(p.y + idx, m);
        }
    }
}

// Output sizes from a descriptor; false when the descriptor is not a pooling the kernels implement.
inline bool pool_fill_args(const paella_pool_desc* d, const float* x, float* y, uint32_t job_id, void* notifier, PoolArgs* a) {
    if (!d || d->C <= 0 || d->H <= 0 || d->W <= 0 || d->R <= 0 || d->S <= 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->pad_h < 0 ||
        d->pad_w < 0 || d->pad_h * 2 > d->R || d->pad_w * 2 > d->S)
        return false;
    const int P = paella_pool_out(d->H, d->R, d->stride_h, d->pad_h, d->ceil_mode);
    const int Q = paella_pool_out(d->W, d->S, d->stride_w, d->pad_w, d->ceil_mode);
    if (P <= 0 || Q <= 0) return false;
    a->x = x; a->y = y;
    a->C = d->C; a->H = d->H; a->W = d->W; a->P = P; a->Q = Q; a->R = d->R; a->S = d->S;
    a->sh = d->stride_h; a->sw = d->stride_w; a->ph = d->pad_h; a->pw = d->pad_w;
    a->is_avg = d->is_avg; a->count_include_pad = d->count_include_pad;
    a->job_id = job_id;
    a->hook_blocks = 0;
    a->notifier = reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier);
    {
        const unsigned long long elements = (unsigned long long)d->C * P * Q, rows = (unsigned long long)d->C * P;
        const unsigned long long x_bytes = (unsigned long long)d->C * d->H * d->W * 4;
        const bool window = (d->R == 3 && d->S == 3) || (d->R == 2 && d->S == 2);
        // the last window starts inside the image or its leading padding, so that clamping stays within the window
        const bool starts_inside = (P - 1) * d->stride_h - d->pad_h < d->H && (Q - 1) * d->stride_w - d->pad_w < d->W;
        a->fast = window && starts_inside && elements * (unsigned long long)Q < (1ull << 32) && rows * (unsigned long long)P < (1ull << 32) &&
                  elements < (1u << 23) && (unsigned long long)d->C * d->H < (1u << 23) && d->W < (1 << 23) && x_bytes < (1ull << 30) ? 1 : 0;
        auto magic = [](unsigned dv, unsigned* mul, unsigned* one) {
            if (dv <= 1) { *mul = 0u; *one = 0xFFFFFFFFu; }
            else { *mul = (unsigned)((1ull << 32) / dv) + 1u; *one = 0u; }
        };
        magic((unsigned)Q, &a->div_q_mul, &a->div_q_one);
        magic((unsigned)P, &a->div_p_mul, &a->div_p_one);
        a->x_bytes = (unsigned)(x_bytes < 0xFFFFFFFFull ? x_bytes : 0xFFFFFFFFull);
        a->out_bytes = (unsigned)(elements * 4 < 0xFFFFFFFFull ? elements * 4 : 0xFFFFFFFFull);
    }
    return true;
}

}  // namespace paella
