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

// Output element number idx (channel-major, then row, then column); does nothing past the last element.
__device__ __forceinline__ void pool_element(const PoolArgs& p, const int idx) {
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
    return true;
}

}  // namespace paella
