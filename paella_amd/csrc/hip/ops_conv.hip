// conv2d for gfx950 (fp32, NCHW, batch 1): implicit GEMM on the fp32 MFMA pipe and a depthwise kernel.
//
// GEMM view:  Y[m][n] = sum_k Wt[m][k] * X~[k][n]   with m = output channel, n = output pixel (p*Q+q),
// k = (c, r, s).  Output pixels of one channel are contiguous in NCHW, so the MFMA "column" index is the
// pixel: operand loads of X~ and stores of Y are unit-stride across the 32 lanes of a half wave.
//
// One wave owns a (32*MI) x (32*NI) output tile and a contiguous slice of the reduction; the KW waves of a
// workgroup share the tile and split k, then add their partial tiles through LDS in fixed wave order
// (deterministic) before the fused epilogue bias -> residual -> activation -> store.
//
// Operand feeding (v_mfma_f32_32x32x2_f32; lane l supplies A[l%32][l/32] and B[l/32][l%32]):
//   * weights are pre-packed on the host as float4 groups [k/4][m][4], so lane (i, kk) fetches the four
//     k values {8c + 4kk + t} of row i with one 16-byte load and a half wave reads 512 contiguous bytes;
//   * the im2col operand is gathered straight from the activation tensor with raw buffer loads whose
//     out-of-range offsets return 0: padding taps, the k tail and the pixel tail need no branches.  Each
//     workgroup first builds, in LDS, the table k -> {byte offset c*H*W + r*dil*W + s*dil, (r*dil) << 16 | (s*dil)}
//     for its slice of the reduction;
//   * when C is a multiple of 8 the reduction index is ordered k = (r, s, c) instead ("tap-major"): the 8 values
//     of a chunk then share one filter tap and differ only in the channel, so the address is a few additions on
//     wave-uniform running counters, the bounds test is done once per chunk instead of once per value, and
//     neither table nor LDS staging nor the barrier after it is needed: the first loads leave right away.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <type_traits>
#include <mutex>
#include <vector>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>

#include "paella_ops.h"
#include <llis/job/finished_block_notifier.h>

#include "launch.h"
#include "out_store.h"
#include "pool_body.h"
#include "dense_body.h"
#include "pack.h"

#ifdef PAELLA_CONV_TIMELINE
// Measurement build only: every wave of a conv leaves sixteen realtime-counter samples (100 MHz) in this buffer.
__device__ unsigned long long* g_tl_buf = nullptr;
__device__ unsigned g_tl_cap = 0;
#define TL_STAMP(i)                           \
    do {                                      \
        __builtin_amdgcn_sched_barrier(0);    \
        tl[i] = (unsigned)wall_clock64();     \
        __builtin_amdgcn_sched_barrier(0);    \
    } while (0)
extern "C" int paella_conv_timeline_set(void* buf, unsigned waves) {
    if (hipError_t e = hipMemcpyToSymbol(HIP_SYMBOL(g_tl_buf), &buf, sizeof(buf))) return (int)e;
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_tl_cap), &waves, sizeof(waves));
}
#else
#define TL_STAMP(i)
#endif

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Quotient by a divisor the host knows: floor(a / d) = umulhi(a, mul) + (a & one) with mul = floor(2^32 / d) + 1 and
// one = 0, exact while a * d < 2^32 (the error term a * (mul * d - 2^32) / (d * 2^32) stays below 1 / d); d = 1 is
// mul = 0, one = ~0.  A division costs about 25 dependent instructions per wave, and the kernel starts with six.
struct FastDiv {
    unsigned mul, one;
};

struct ConvArgs {
    const float* x;
    const float4* wpk;
    const float* bias;
    const float* residual;
    const float* slope;
    float* y;
    int H, W, Q, PQ;
    int sh, sw, ph, pw;
    int K, m_pad, nchunks;
    int kdim, RS, S, dh, dw;        // reduction length C*R*S, filter plane R*S, filter width, dilations
    int CB;                         // tap-major order only: chunks per filter tap (C / 8)
    unsigned w_bytes;               // size of the packed weights
    int splits, chunks_per_split;   // grid-level split of the reduction
    int n_tiles_n, n_tiles_m;       // output tiles along pixels and along channels; the grid is 1-D over n*m*splits
    int slab_major;                 // which workgroups share an XCD: 1 = same weights, 0 = neighbouring pixels
    float* ws_partials;             // [tile][split][NACC][64] partial tiles (request-private workspace)
    unsigned* ws_counters;          // [tile] arrival counters, zero between launches
    unsigned x_bytes;
    int act;
    float lo, hi;
    uint32_t job_id;
    unsigned hook_blocks;           // workgroups of this launch that report to `notifier`; 0: all of them (one job per launch)
    llis::job::FinishedBlockNotifier* notifier;
    // divisors: of the work-list position (pixel tiles per slab, or slabs per pixel tile), channel tiles, output width,
    // chunks per filter tap, filter width; fast_div = 0: operands too large for the shortcut, divide
    FastDiv div_w, div_tm, div_q, div_cb, div_s;
    int fast_div;
    int pointwise;                  // tap-major only: 1x1 filter, stride 1, no padding
    int pair_s0;                    // tap-major, 3-wide stride-2 filters: first of the two paired filter columns, or -1 (see load_frag)
};

// The quotient for dividends and divisors the host has checked; where it could not, the kernel divides (ConvArgs::fast_div).
__device__ __forceinline__ unsigned quot_fast(unsigned a, const FastDiv& f) { return __umulhi(a, f.mul) + (a & f.one); }

__device__ __forceinline__ float apply_act(float v, int act, float slope, float lo, float hi) {
    switch (act) {
        case PAELLA_ACT_RELU:  return fmaxf(v, 0.f);
        case PAELLA_ACT_RELU6: return fminf(fmaxf(v, 0.f), 6.f);
        case PAELLA_ACT_PRELU: return v > 0.f ? v : v * slope;
        case PAELLA_ACT_CLIP:  return fminf(fmaxf(v, lo), hi);
        default:               return v;
    }
}

template <int MI, int NI>
struct Frag {
    float4 a[MI];
    float b[NI][4];
    float4 sc, sh;  // only with a fused input transform: scale and shift of the lane's four channels (zero for a padding tap)
};

// Per-channel transform of the conv's input, applied to the im2col operand on its way into the matrix pipe:
// x' = max(x * scale[c] + shift[c], lo) inside the image, 0 in the padding -- a batch-norm (lo = -inf) or batch-norm + ReLU
// (lo = 0) stage that would otherwise run as a kernel of its own in front of the conv.
struct PreOp {
    const float* scale;
    const float* shift;
    float lo;
};

// One workgroup's share of a conv: output tile and reduction split number `bid` of the problem `p`.
// PW ("pointwise"): a 1x1 filter with stride 1 and no padding in tap-major order -- an input pixel is its output pixel, there
// are no taps to step through and nothing to test per tap.
// PRE: kPreBounded with a lower bound (ReLU), kPreUnbounded without (a batch-norm alone: the four maxima per chunk are not
// computed at all -- a vector instruction costs a sixteenth of a matrix instruction of pipe time).
constexpr int kPreNone = 0, kPreBounded = 1, kPreUnbounded = 2;
template <int MI, int NI, int KW, bool TAP_MAJOR, int PRE = kPreNone, int DEPTH = 0, bool PW = false>
__device__ __forceinline__ void conv_tile(const ConvArgs& p, const unsigned bid, const PreOp pre = PreOp{nullptr, nullptr, 0.f}) {
    static_assert(!PRE || (TAP_MAJOR && MI * NI == 1), "the input transform is built for the smallest tile in tap-major order");
    static_assert(!PW || TAP_MAJOR, "the pointwise shortcut belongs to the tap-major order");
    // A grouped launch starts every conv at a multiple of eight workgroups (see align_start): the ids between the end of one
    // problem and the start of the next belong to no tile and report to nobody.
#ifdef PAELLA_CONV_TIMELINE
    unsigned tl[16] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};  // low words: a launch is over long before they wrap (43 s)
#endif
    TL_STAMP(0);
    // The fields the prologue uses, requested together and waited for once.  Read where they are used, each costs a trip to
    // the scalar cache of its own, one after the other -- some twenty of them before a wave's first operand load.  (Only where
    // the scalar registers are there for it: the eight-wave small tile, which is what nearly every launch runs.)
    // ... and held in scalar registers until the prologue is through with them: as results of an (empty) asm statement the
    // compiler cannot fetch them again where they are used, which it otherwise does, one trip each.
    struct Held {
        int n_tiles_n, n_tiles_m, splits, slab_major, fast_div;
        FastDiv div_w, div_tm;
    } a;
    a.n_tiles_n = p.n_tiles_n; a.n_tiles_m = p.n_tiles_m; a.splits = p.splits; a.slab_major = p.slab_major; a.fast_div = p.fast_div;
    a.div_w = p.div_w; a.div_tm = p.div_tm;
    if (KW == 8 && MI * NI == 1 && DEPTH == 0) {
        const unsigned long long a0 = (unsigned long long)p.x, a1 = (unsigned long long)p.wpk, a2 = (unsigned long long)p.notifier;
        asm volatile("" ::"s"(a0), "s"(a1), "s"(a2), "s"(p.H), "s"(p.W), "s"(p.Q), "s"(p.PQ), "s"(p.sh), "s"(p.sw), "s"(p.ph), "s"(p.pw), "s"(p.m_pad),
                     "s"(p.nchunks), "s"(p.CB), "s"(p.w_bytes), "s"(p.chunks_per_split), "s"(p.x_bytes), "s"(p.job_id), "s"(p.hook_blocks),
                     "s"(p.div_q.mul), "s"(p.div_q.one));
        asm volatile("" : "+s"(a.n_tiles_n), "+s"(a.n_tiles_m), "+s"(a.splits), "+s"(a.slab_major), "+s"(a.fast_div), "+s"(a.div_w.mul), "+s"(a.div_w.one),
                     "+s"(a.div_tm.mul), "+s"(a.div_tm.one));
    }
    TL_STAMP(8);
    if (bid >= (unsigned)(a.n_tiles_n * a.n_tiles_m * a.splits)) return;
    const unsigned hook_blocks = p.hook_blocks ? p.hook_blocks : gridDim.x;
    paella::hook_entry(p.notifier, p.job_id, hook_blocks);
    // Waves of this workgroup whose result stores have been acknowledged (see the end of this function); cleared here, and
    // the barrier of the cross-wave sum lies between this store and the first increment.
    __shared__ unsigned waves_done;

    // One LDS region, used first for the k -> offset table and, after the reduction loop, for the partial tiles.
    extern __shared__ __align__(16) char smem[];
    int2* ltab = reinterpret_cast<int2*>(smem);
    float* red = reinterpret_cast<float*>(smem);
    // With a fused input transform, behind the partial tiles' region (waves leave the loop at different times): 64 bytes of zeros,
    // then per four input channels their four scales and their four shifts, 32 bytes.
    char* const ptab = smem + (KW > 1 ? KW * MI * NI * 16 * 64 * 4 : 0);
    // A thread's first two entries of that table are requested here, so that they travel while the tile is decoded (entries
    // past the last channel read as zero and are not written).
    constexpr int kPreEarly = 2;
    float pre_early_s[kPreEarly], pre_early_h[kPreEarly];
    if (PRE) {
        const unsigned len = (unsigned)p.CB * 32u;
        const __amdgpu_buffer_rsrc_t sr = __builtin_amdgcn_make_buffer_rsrc((void*)pre.scale, 0, len, 0x00027000);
        const __amdgpu_buffer_rsrc_t hr = __builtin_amdgcn_make_buffer_rsrc((void*)pre.shift, 0, len, 0x00027000);
#pragma unroll
        for (int e = 0; e < kPreEarly; ++e) {
            const int off = ((int)threadIdx.x + e * 64 * KW) * 4;
            pre_early_s[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sr, off, 0, 0));
            pre_early_h[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(hr, off, 0, 0));
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, and the compiler may know it
    if (KW > 1 && wave == 0) waves_done = 0;  // every lane of the first wave stores the same zero: no compare on the vector unit
    // One lane of the workgroup, tested afresh at each use: held from the first use to the last, the lane mask costs two scalar
    // registers that the loop has no room for (they went to a vector register's lanes and back, a vector instruction each way).
    auto first_thread = [&]() {
        int l = lane, w = wave;
        asm volatile("" : "+v"(l), "+s"(w));
        return w == 0 && l == 0;
    };
    const int j = lane & 31;
    const int kk = lane >> 5;
    // 0 or -1 (one signed bit-field extract): a product of kk and a wave-uniform value is then one `and` (a 32-bit vector
    // multiply takes four passes)
    const int negkk = (int)((unsigned)lane << 26) >> 31;
    // Workgroup -> (pixel tile, channel tile, reduction split).  Workgroup ids go round-robin over the eight
    // XCDs, each with its own L2; the ids that land on one XCD are given a contiguous run of the work list, and
    // the list is ordered so that a run shares what the layer reads most of: the same slab of weights (layers
    // with small feature maps) or neighbouring pixel tiles, whose 3x3 halos overlap (layers with large ones).
    int tile_n, tile_m, split;
    {
        const unsigned total = (unsigned)(a.n_tiles_n * a.n_tiles_m * a.splits);
        const unsigned xcd = bid & 7u, j = bid >> 3;
        const unsigned q = total >> 3, r = total & 7u;
        const unsigned w = a.slab_major == 2 ? bid : xcd * q + (xcd < r ? xcd : r) + j;  // 2: plain order (experiments)
        // Both orders are one division of the work-list position and one of its quotient or remainder, so the order only selects
        // (scalar selects, no branch; branches here came out as a flag in a vector register tested on the vector unit).
        auto decode = [&](auto div) {
            const bool slabs = a.slab_major != 0;
            const unsigned d_w = slabs ? (unsigned)a.n_tiles_n : (unsigned)(a.n_tiles_m * a.splits);
            const unsigned q = div(w, d_w, a.div_w);
            const unsigned r = w - q * d_w;
            const unsigned rest = slabs ? q : r;  // slab number (channel tile and split), or position within the pixel tile's share
            tile_n = (int)(slabs ? r : q);
            split = (int)div(rest, (unsigned)a.n_tiles_m, a.div_tm);
            tile_m = (int)(rest - (unsigned)split * (unsigned)a.n_tiles_m);
        };
        // (readfirstlane: the compiler takes the result of an asm statement for a per-lane value and would test it on the vector unit)
        if (__builtin_amdgcn_readfirstlane(a.fast_div)) decode([](unsigned x, unsigned, const FastDiv& f) { return quot_fast(x, f); });
        else decode([](unsigned x, unsigned d, const FastDiv&) { return x / d; });
    }
    const int m0 = tile_m * (32 * MI);
    const int n0 = tile_n * (32 * NI);
    TL_STAMP(9);

    // The input through a descriptor that starts pad_off bytes in front of the tensor, pad_off = (pad_h * W + pad_w) * 4: a lane's
    // offset is then that of input element (ho * stride_h, wo * stride_w) -- never negative, so a filter tap's offset
    // (r * dil_h * W + s * dil_w) * 4 can ride in the loads' scalar offset and the lane's part need not change with the tap.
    const unsigned pad_off = TAP_MAJOR ? (unsigned)(p.ph * p.W + p.pw) * 4u : 0u;
    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)(reinterpret_cast<const char*>(p.x) - pad_off), 0, p.x_bytes + pad_off, 0x00027000);

    const unsigned plane = (unsigned)p.PQ * 4u;  // bytes of one output channel
    // A lane's offset within its tile's output channels (see the output addressing below), one per pixel tile, computed once and held (as the result of an empty asm
    // statement: the compiler otherwise works it out again at each of its four uses, four vector instructions a time).
    int lane_offs[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int pix = n0 + ni * 32 + j;
        lane_offs[ni] = pix < p.PQ ? (int)((unsigned)(negkk & (int)(4u * plane)) + (unsigned)pix * 4u) : (int)0x80000000u;
        asm volatile("" : "+v"(lane_offs[ni]));
    }
    const int HW4 = p.H * p.W * 4;
    const int kk4hw = negkk & (4 * HW4);
    int hb[NI], wb[NI], base[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int pix = n0 + ni * 32 + j;
        if (PW) {  // input pixel = output pixel
            hb[ni] = wb[ni] = 0;
            base[ni] = lane_offs[ni];  // H * W = P * Q here: the same offset, out of range (negative) past the last pixel
            continue;
        }
        const int ho = __builtin_amdgcn_readfirstlane(a.fast_div) ? (int)quot_fast((unsigned)pix, p.div_q) : (int)((unsigned)pix / (unsigned)p.Q);
        const int wo = pix - __mul24(ho, p.Q);  // every factor here is a pixel coordinate or an extent: far below 2^23
        hb[ni] = (pix < p.PQ) ? __mul24(ho, p.sh) - p.ph : -0x100000;
        wb[ni] = __mul24(wo, p.sw) - p.pw;
        base[ni] = (__mul24(hb[ni], p.W) + wb[ni]) * 4 + (TAP_MAJOR ? (int)pad_off + kk4hw : 0);
    }
    TL_STAMP(10);

    // Reduction range of this workgroup (grid-level split), then of this wave inside it.
    const int g_begin = split * p.chunks_per_split;
    const int g_end = min(p.nchunks, g_begin + p.chunks_per_split);
    const int cpw = (int)((unsigned)(g_end - g_begin + KW - 1) / (unsigned)KW);  // the plan leaves no split empty: never negative
    const int c_begin = g_begin + wave * cpw;
    const int c_end = min(g_end, c_begin + cpw);

    // Not zeroed here: the first matrix instruction of a wave's first chunk takes a constant zero as its addend (sixteen vector
    // moves per wave less; a vector instruction costs matrix-pipe time, and a wave that sits in its prologue while others are in
    // their loops waits for the pipe once per vector instruction).  Only a wave without any chunk zeroes them explicitly.
    f32x16 acc[MI][NI];

    // Chunks outside [c_begin, c_end) are requested at an out-of-range offset: the loads keep their place in
    // the (static) issue order, return zeros and touch no memory.
    __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc((void*)p.wpk, 0, p.w_bytes, 0x00027000);
    // Vector instructions take their four cycles out of the matrix pipe's time on this part (a matrix instruction and a vector
    // instruction of any wave of the SIMD do not overlap), so the per-chunk address arithmetic is kept on the scalar unit:
    // a lane's part of an offset sits in a register that changes only when the filter tap does, the chunk's part rides in the
    // load's scalar offset (not range-checked: an out-of-range lane offset stays out of range, a valid one stays valid), and a
    // chunk outside the wave's range reads through a descriptor of zero length instead of an offset made invalid per lane.
    // (the same descriptor with length zero: choosing between the two is then one scalar select, on the length word)
    const char* const x_base = reinterpret_cast<const char*>(p.x) - pad_off;
    const unsigned x_len = p.x_bytes + pad_off, w_len = p.w_bytes;
    const int wlane = (int)(((unsigned)(negkk & p.m_pad) + (unsigned)(m0 + j)) * 16u);
    const int wstep = p.m_pad * 32;  // bytes of weights per chunk and row block: two reduction steps of m_pad rows of 16 bytes
    int tap_voff[NI];
    bool tap_ok[NI];
    // With a fused input transform: what a lane keeps of a chunk's table address -- everything in the second half of the wave,
    // all but the bit that selects the second reduction step's four channels in the first, nothing (the zeros in front of the
    // table) where the lane's pixel or tap is padding.  It changes only when the tap does.
    int pre_sel = (PRE && PW) ? (base[0] >= 0 ? (negkk | ~32) : 0) : 0;
    bool tap_stale = true;
    int tap_off = 0;  // byte offset of the current filter tap, wave-uniform
    // Paired filter columns (stride 2 across a 3-wide filter, pair_s0 >= 0).  With stride 2 a lane's pixels are every other
    // element of a line, so each line fetched delivers half as many operands.  Two neighbouring filter columns read
    // neighbouring input pixels: for their chunks the half wave selects the COLUMN instead of four more channels -- lane (j, kk)
    // reads pixel 2 q_j + kk, the 64 lanes of a load cover 64 consecutive elements -- and a chunk holds four channels of both
    // columns.  The host packs the weights to match: per filter row, CB chunks of the unpaired column (eight channels each), then
    // 2 CB chunks of the pair (four channels of both columns each), so a row is 3 CB chunks either way and chunk c is still
    // (unit c / CB, block c % CB).  The host has checked that both columns lie inside the image for every output pixel.
    const int pair_s0 = (TAP_MAJOR && !PW && MI * NI == 1) ? p.pair_s0 : -1;
    const int pair_delta = (negkk & (p.dw * 4)) - kk4hw;  // from the lane's offset for a plain chunk to that for a paired one
    int seg_chan0 = 0, seg_chans = 8;  // first channel of the current unit's chunks, channels per chunk; wave-uniform
    bool seg_pair = false;
    auto load_frag = [&](int c, bool valid, Frag<MI, NI>& f) {
        if (TAP_MAJOR) {
            const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void*)p.wpk, 0, valid ? w_len : 0u, 0x00027000);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const auto v = __builtin_amdgcn_raw_buffer_load_b128(wr, wlane, c * wstep + mi * 32 * 16, 0);
                f.a[mi] = __builtin_bit_cast(float4, v);
            }
            // Where chunk c lies: filter tap and channel block within it, all on the scalar unit (two multiply-highs; a running
            // position with carries from block to column to row ended up in vector registers).
            int cb = c, tap_soff = 0;
            if (!PW) {
                const int tap = (int)quot_fast((unsigned)c, p.div_cb);
                cb = c - tap * p.CB;
                if (tap_stale | (cb == 0)) {  // wave-uniform: once per filter tap
                    const int r = (int)quot_fast((unsigned)tap, p.div_s);
                    int col = tap - r * p.S;  // the filter column, or with paired columns the unit's place in its row
                    seg_pair = false;
                    seg_chan0 = 0;
                    seg_chans = 8;
                    if (pair_s0 >= 0) {
                        seg_pair = col != 0;                     // places 1 and 2: the two halves of the pair's chunks
                        seg_chan0 = col == 2 ? p.CB * 4 : 0;
                        seg_chans = seg_pair ? 4 : 8;
                        col = seg_pair ? pair_s0 : 2 - 2 * pair_s0;  // the pair's first column; the unpaired one is 2 or 0
                    }
                    const int dy = r * p.dh, dx = col * p.dw;
                    tap_off = (dy * p.W + dx) * 4;
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        tap_ok[ni] = ((unsigned)(hb[ni] + dy) < (unsigned)p.H) & ((unsigned)(wb[ni] + dx) < (unsigned)p.W);
                        tap_voff[ni] = tap_ok[ni] ? base[ni] : -1;
                    }
                    if (seg_pair) {
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) tap_voff[ni] = tap_ok[ni] ? base[ni] + pair_delta : -1;
                    }
                    if (PRE) pre_sel = tap_ok[0] ? (seg_pair ? -1 : (negkk | ~32)) : 0;  // a pair's chunk: the same four channels in both halves
                    tap_stale = false;
                }
                tap_soff = tap_off;
            }
            const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)x_base, 0, valid ? x_len : 0u, 0x00027000);
            const int chan0 = PW ? cb * 8 : seg_chan0 + cb * seg_chans;  // first channel of the chunk
            const int chunk_off = chan0 * HW4 + tap_soff;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int voff = PW ? base[ni] : tap_voff[ni];
#pragma unroll
                for (int t = 0; t < 4; ++t) f.b[ni][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, voff, chunk_off + t * HW4, 0));
                if (PRE) {
                    // Scale and shift of the lane's four channels, from the table in LDS: requested through the vector cache like
                    // the operands, their 2 KB per wave and chunk doubled what the cache has to deliver and cost a fifth of the
                    // kernel's rate with the device full.  Where the lane's pixel or tap is padding, and for a chunk past the
                    // wave's range, the address is that of the zeros, and the zero that the operand load returned stays the
                    // zero the padding asks for.  One vector instruction: the chunk's part of the address is wave-uniform.
                    const int chunk_addr = valid ? ((64 + chan0 * 8) | ((!PW && seg_pair) ? 0 : 32)) : 0;
                    const char* const e = ptab + (pre_sel & chunk_addr);
                    f.sc = *reinterpret_cast<const float4*>(e);
                    f.sh = *reinterpret_cast<const float4*>(e + 16);
                }
            }
            return;
        }
        const int woff = valid ? (int)((((unsigned)(c * 2 + kk) * (unsigned)p.m_pad) + (unsigned)(m0 + j)) * 16u) : -1;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const auto v = __builtin_amdgcn_raw_buffer_load_b128(wres, woff, mi * 32 * 16, 0);
            f.a[mi] = __builtin_bit_cast(float4, v);
        }
        const int4* t = reinterpret_cast<const int4*>(ltab + ((valid ? c : g_begin) - g_begin) * 8 + kk * 4);
        const int4 t0 = t[0], t1 = t[1];
        const int off[4] = {t0.x, t0.z, t1.x, t1.z};
        const int rs[4] = {t0.y, t0.w, t1.y, t1.w};
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int h = hb[ni] + (rs[t] >> 16);
                const int w = wb[ni] + (rs[t] & 0xFFFF);
                const bool ok = valid & ((unsigned)h < (unsigned)p.H) & ((unsigned)w < (unsigned)p.W);
                const int voff = ok ? base[ni] + off[t] : -1;
                f.b[ni][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xres, voff, 0, 0));
            }
        }
    };

    // Build this workgroup's slice of the k -> offset table in LDS (a few entries per thread, arithmetic only).
    if (!TAP_MAJOR) {
        const int n_entries = (g_end - g_begin) * 8;
        for (int i = threadIdx.x; i < n_entries; i += 64 * KW) {
            const int k = g_begin * 8 + i;
            const int c = k / p.RS;
            const int rem = k - c * p.RS;
            const int r = rem / p.S;
            const int sx = rem - r * p.S;
            int2 e;
            e.x = c * HW4 + (r * p.dh * p.W + sx * p.dw) * 4;
            e.y = ((r * p.dh) << 16) | (sx * p.dw);
            if (k >= p.kdim) e = make_int2(0, 0x7FFF0000);  // row far outside the image: the tap reads as zero
            ltab[i] = e;
        }
        __syncthreads();
    }
    // The table of scales and shifts of a fused input transform: every input channel's, a few entries per thread.
    if (PRE) {
        const int n_chan = p.CB * 8;
        const __amdgpu_buffer_rsrc_t sr = __builtin_amdgcn_make_buffer_rsrc((void*)pre.scale, 0, (unsigned)n_chan * 4u, 0x00027000);
        const __amdgpu_buffer_rsrc_t hr = __builtin_amdgcn_make_buffer_rsrc((void*)pre.shift, 0, (unsigned)n_chan * 4u, 0x00027000);
        if (threadIdx.x < 16) reinterpret_cast<float*>(ptab)[threadIdx.x] = 0.f;
        auto entry = [&](int i) { return reinterpret_cast<float*>(ptab + 64 + (i >> 2) * 32 + (i & 3) * 4); };
#pragma unroll
        for (int e = 0; e < kPreEarly; ++e) {
            const int i = (int)threadIdx.x + e * 64 * KW;
            if (i < n_chan) {
                entry(i)[0] = pre_early_s[e];
                entry(i)[4] = pre_early_h[e];
            }
        }
        for (int i = (int)threadIdx.x + kPreEarly * 64 * KW; i < n_chan; i += 64 * KW) {
            entry(i)[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sr, i * 4, 0, 0));
            entry(i)[4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(hr, i * 4, 0, 0));
        }
        __syncthreads();
    }
    // Drain every earlier vector-memory operation (the start hook's store among them) once, here: with a
    // store still pending the compiler must assume out-of-order completion and would make every wait in
    // the pipelined loop below a full vmcnt(0).
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched

    constexpr int NACC = MI * NI * 16;
    constexpr int RPW = NACC / KW;
    // (a variant with a deeper operand pipeline keeps its registers for the chunks in flight)
    // (nor does the variant with an input transform: its scale and shift operands take the registers, and with the epilogue's
    // operands requested after the loop it fits the 64 registers of eight waves per SIMD)
    constexpr bool kPrefetchEpilogue = !PRE && (DEPTH ? RPW <= 4 : RPW <= 16);
    // Output addressing.  Register r of the tile (r = wave * RPW + rr for this wave) holds, in lane (j, kk), output channel
    // m0 + row(r) + 4 * kk at pixel n0 + 32 * ni(r) + j.  Everything that depends on the tile, the wave or r is wave-uniform and
    // goes into buffer descriptors and scalar offsets built on the scalar unit: per tensor a descriptor at the tile's first
    // channel that ends at channel K, per register the row's byte offset as the access's scalar offset.  A lane contributes one
    // byte offset per pixel tile -- its pixel within a channel plane plus the four planes of its half wave, or an offset beyond
    // any length for a pixel past P*Q -- and the hardware holds the sum against the descriptor's length: rows at or past K and
    // pixels past P*Q read as zero and their stores are dropped, without a compare on the vector unit.
    // (K * P * Q * 4 < 2^31 is a condition of the plan.)
    auto row_of = [&](int w, int rr) {
        const int r = w * RPW + rr;
        const int e = r & 15;
        return ((r >> 4) / NI) * 32 + (e >> 2) * 8 + (e & 3);
    };
    auto lane_off = [&](int rr) { return lane_offs[((wave * RPW + rr) >> 4) % NI]; };
    const int rows_tile = max(p.K - m0, 0);  // channels from this tile's first one to the last that exists (may exceed the tile)
    const float* const res_tile = p.residual ? p.residual + (size_t)m0 * p.PQ : nullptr;
    float* const y_tile = p.y + (size_t)m0 * p.PQ;
    // The hardware tests lane offset >= length - scalar offset (unsigned), so the length is that of all the tile's channels and
    // a row's scalar offset is held at that length: the difference is then zero for a row that does not exist and every lane of
    // the access is out of range (an offset past the length would wrap the difference and pass the test).  One descriptor per
    // tensor; what changes with the register is a scalar offset of two instructions.
    const unsigned tile_len = (unsigned)rows_tile * plane;
    const unsigned chan_len = (unsigned)rows_tile * 4u;
    // An operand that is not there (no bias, no residual) is read through a descriptor of length zero: zeros without a branch, a
    // register move and a memory access.
    auto plane_rsrc = [&](const float* tile_base, int) { return __builtin_amdgcn_make_buffer_rsrc((void*)tile_base, 0, tile_base ? tile_len : 0u, 0x00027000); };
    auto chan_rsrc = [&](const float* per_channel, int) {  // bias, slope: one float per channel
        // (the base as an integer sum: arithmetic on a null pointer would let the compiler conclude that it is not null)
        return __builtin_amdgcn_make_buffer_rsrc((void*)((uintptr_t)per_channel + (uintptr_t)m0 * 4u), 0, per_channel ? chan_len : 0u, 0x00027000);
    };
    // Worked out twice, before the loop for the operands requested there and again after it (from a wave number the compiler
    // cannot tell is the same): held across the loop, these scalars had no register left and went to a vector register's lanes
    // and back -- a vector instruction and a wait each way, where a dozen scalar instructions do.
    struct RowOffsets {
        int plane[RPW], chan[RPW];
    };
    auto row_offsets = [&](int w) {
        RowOffsets o;
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            o.plane[rr] = (int)min((unsigned)row_of(w, rr) * plane, tile_len);
            o.chan[rr] = (int)min((unsigned)row_of(w, rr) * 4u, chan_len);
        }
        return o;
    };
    const int chan_voff = negkk & 16;
    // The wave finally owns RPW of the tile's NACC accumulator registers (summed over the KW waves).  Request
    // the epilogue's operands for them now, so that their latency hides behind the reduction loop.
    // (requested once the first chunks' operand loads are out: the loop cannot start before those arrive)
    float bias_v[RPW], res_v[RPW];
    auto prefetch_epilogue = [&]() {
        if (!kPrefetchEpilogue) return;
        const RowOffsets o = row_offsets(wave);
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            bias_v[rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(chan_rsrc(p.bias, rr), chan_voff, o.chan[rr], 0));
            res_v[rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(plane_rsrc(res_tile, rr), lane_off(rr), o.plane[rr], 0));
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // Software pipeline of depth D: D chunks of operands are in flight per wave; each slot is refilled with
    // the chunk D ahead right after it has been consumed.  Shallow is better here: the small tile measured
    // fastest at depth 2, alone (6.1 us for the 64-channel 56x56 layer against 6.4 at depth 4) and with many
    // kernels in flight (2.4 against 2.7 us per kernel): fewer registers, so four workgroups fit a CU, and other
    // waves hide the latency that a deeper pipeline would.  Three slots with the refill issued ahead of the current
    // chunk's matrix instructions were no better either (23.8 against 24.9 TFLOP/s over a ResNet-18 pass): the loop is
    // bound by what the compute unit's vector cache can take in -- each wave fetches its own 32 x 8 operand
    // fragments, 147 KB per workgroup for a 64-channel 3x3 layer -- not by exposed latency.  (Again once the kernel had shrunk to
    // 44 registers, so that depth 3 and 4 fit eight waves per SIMD at 52 and 60: 76.8 and 76.4 against 78.1 TFLOP/s with the
    // device full.  Requesting one input dword per chunk instead of four -- wrong results, timing only -- gives 84 against 77:
    // the load path is worth at most 9 % here, and half again on the stride-2 layers, whose lanes use every other pixel of a line.)
    constexpr int D = DEPTH ? DEPTH : (MI * NI == 1) ? 2 : 4;
    // first: the accumulators hold nothing yet, the first matrix instruction into each takes zero as its addend
    auto compute = [&](const Frag<MI, NI>& f, auto first) {
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const float av = t == 0 ? f.a[mi].x : t == 1 ? f.a[mi].y : t == 2 ? f.a[mi].z : f.a[mi].w;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    float bv = f.b[ni][t];
                    if (PRE) {
                        const float sc = t == 0 ? f.sc.x : t == 1 ? f.sc.y : t == 2 ? f.sc.z : f.sc.w;
                        const float sh = t == 0 ? f.sh.x : t == 1 ? f.sh.y : t == 2 ? f.sh.z : f.sh.w;
                        bv = bv * sc + sh;  // the padding's 0 * 0 + 0 stays 0, also under a bound of 0
                        if (PRE == kPreBounded) bv = fmaxf(bv, pre.lo);
                    }
                    if (decltype(first)::value && t == 0) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, zero, 0, 0, 0);
                    else acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[mi][ni], 0, 0, 0);
                }
            }
        }
    };
    constexpr std::true_type kFirst{};
    constexpr std::false_type kLater{};
    // (Raising the wave's priority for the loop, s_setprio 2, or from the loop to the end of the kernel, s_setprio 3, changed
    // nothing alone and nothing or -10 % with four passes in flight: 15.8 / 14.2 / 15.8 thousand ResNet-18 passes per second.
    // The opposite, priority 3 outside the loop so that prologues and epilogues get their few vector instructions in between
    // other waves' matrix instructions: +2 % with the device full while a wave still executed some 130 vector instructions
    // around its loop, -1 % everywhere once those were down to about 70; at 56: priority 2 from entry to the first operand
    // requests -4 % with the device full and -2 % served, priority for the loop, for the epilogue or for both within +-0.5 %.)
    TL_STAMP(1);
    if (c_begin < c_end) {
        Frag<MI, NI> frag[D];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            load_frag(c_begin + d, c_begin + d < c_end, frag[d]);
            __builtin_amdgcn_sched_barrier(0);  // same issue order as in the steady state
#ifdef PAELLA_CONV_TIMELINE
            if (d < 2) TL_STAMP(11 + d);
#endif
        }
        prefetch_epilogue();
        TL_STAMP(2);
        const int n = c_end - c_begin;
        const int c_main_end = c_begin + (n / D) * D;
        // One group of D chunks: each slot is consumed and refilled with the chunk D ahead.
        auto group = [&](int c, auto first) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                if (d == 0) compute(frag[d], first);
                else compute(frag[d], kLater);
#ifdef PAELLA_CONV_TIMELINE
                if (d == 0 && decltype(first)::value) {
                    __builtin_amdgcn_sched_barrier(0);
                    TL_STAMP(3);
                }
#endif
                // keep the refill of this slot right here: hoisting all loads to one place would make every
                // iteration wait for the whole memory latency
                __builtin_amdgcn_sched_barrier(0);
                load_frag(c + D + d, c + D + d < c_end, frag[d]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (n >= D) {
            // Branch-free steady state: whole groups of D chunks, the first one apart (it starts the accumulators).
            group(c_begin, kFirst);
            for (int c = c_begin + D; c < c_main_end; c += D) group(c, kLater);
            // Up to D-1 leftover chunks are already sitting in the first slots.
            const int rest = n - (n / D) * D;
#pragma unroll
            for (int d = 0; d < D - 1; ++d)
                if (d < rest) compute(frag[d], kLater);
        } else {
            // fewer chunks than slots: all of them are sitting in the first slots
            compute(frag[0], kFirst);
#pragma unroll
            for (int d = 1; d < D - 1; ++d)
                if (d < n) compute(frag[d], kLater);
        }
    } else {
        prefetch_epilogue();
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;
    }

    // Finishes the wave's RPW outputs.  Every operand load comes first, then the arithmetic, then the stores back
    // to back: a load between two stores would make the compiler wait for the earlier store as well (one counter
    // covers both), and a write-through store takes about 0.3 us to be acknowledged.
    auto epilogue_all = [&](float (&v)[RPW]) {
        int wave_again = wave;
        asm volatile("" : "+s"(wave_again));
        const RowOffsets o = row_offsets(wave_again);
        const int act = p.act;  // wave-uniform: one scalar branch per kind of activation around straight-line code for all registers
        float sl[RPW];
        if (act == PAELLA_ACT_PRELU) {
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr)
                sl[rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(chan_rsrc(p.slope, rr), chan_voff, o.chan[rr], 0));
        }
        if (!kPrefetchEpilogue) {
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) {
                bias_v[rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(chan_rsrc(p.bias, rr), chan_voff, o.chan[rr], 0));
                res_v[rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(plane_rsrc(res_tile, rr), lane_off(rr), o.plane[rr], 0));
            }
        }
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            v[rr] += bias_v[rr];
            v[rr] += res_v[rr];
        }
        if (act == PAELLA_ACT_RELU) {
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) v[rr] = fmaxf(v[rr], 0.f);
        } else if (act == PAELLA_ACT_RELU6) {
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) v[rr] = fminf(fmaxf(v[rr], 0.f), 6.f);
        } else if (act == PAELLA_ACT_PRELU) {
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) v[rr] = v[rr] > 0.f ? v[rr] : v[rr] * sl[rr];
        } else if (act == PAELLA_ACT_CLIP) {
            const float lo = p.lo, hi = p.hi;
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) v[rr] = fminf(fmaxf(v[rr], lo), hi);
        }
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr)  // write-through (sc1), like store_out
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v[rr]), plane_rsrc(y_tile, rr), lane_off(rr), o.plane[rr], 16);
    };

    TL_STAMP(4);
    float mine[RPW];
    if (KW == 1) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if ((mi * NI + ni) * 16 + e < RPW) mine[(mi * NI + ni) * 16 + e] = acc[mi][ni][e];
    } else {
        if (!TAP_MAJOR) __syncthreads();  // every wave is done with the table before the partial tiles overwrite it
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    red[((wave * NACC) + (mi * NI + ni) * 16 + e) * 64 + lane] = acc[mi][ni][e];
        TL_STAMP(13);
        __syncthreads();
        TL_STAMP(14);
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            float v = red[((0 * NACC) + wave * RPW + rr) * 64 + lane];  // wave order: the sum does not depend on which wave finished first
#pragma unroll
            for (int w = 1; w < KW; ++w) v += red[((w * NACC) + wave * RPW + rr) * 64 + lane];
            mine[rr] = v;
        }
    }

    TL_STAMP(5);
    if (p.splits == 1) {
        epilogue_all(mine);
    } else {
        // Deterministic split-k: every workgroup parks its partial tile in the workspace (write-through),
        // bumps the tile's counter, and the workgroup that arrives last adds the partials in split order and
        // runs the epilogue.  The counter is left at zero for the next launch.
        // Ordering without fences: store_out is a device-scope write-through store, so once s_waitcnt vmcnt(0) has returned
        // the partial tile is in memory, ahead of the counter bump that follows the barrier; the last arriver reads the
        // partials with device-scope atomic loads, which do not hit in its own caches.  A release on the bump and an acquire
        // after it would add a cache write-back and an invalidate per workgroup for data that never sat in a cache.
        // Everything the last arriver needs is read here, ahead of the counter bump, and the arrival number is made wave-uniform
        // for the compiler: fetched again after an atomic inside a one-lane branch, the split count and the pointers counted as
        // per-lane values, and every load through a descriptor built from them was wrapped in a loop over the lanes' values.
        const int nsplits = __builtin_amdgcn_readfirstlane(p.splits);
        const int tile = tile_m * p.n_tiles_n + tile_n;
        unsigned* const counter = p.ws_counters + tile;
        // the tile's partial tiles, [split][NACC][64 lanes]: one descriptor, a lane's offset is its lane number
        float* const partials = p.ws_partials + (size_t)tile * nsplits * (NACC * 64);
        const unsigned partials_len = (unsigned)nsplits * (NACC * 256u);
        const __amdgpu_buffer_rsrc_t pres = __builtin_amdgcn_make_buffer_rsrc((void*)partials, 0, partials_len, 0x00027000);
        const int lane4 = lane * 4;
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, mine[rr]), pres, lane4, (split * NACC + wave * RPW + rr) * 256, 16);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        __shared__ unsigned arrived;
        if (first_thread()) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(arrived) == (unsigned)nsplits - 1) {
            float v[RPW];
#pragma unroll
            for (int rr = 0; rr < RPW; ++rr) v[rr] = 0.f;
            // Partial tiles are requested in batches (eight, then four, two, one: as many as are left, all in flight together) and
            // added in split order: the sum does not depend on which workgroup came last.  Device scope (sc1): they were written
            // by other workgroups and must not come from this one's caches.
            auto add_batch = [&](int z0, auto batch) {
                constexpr int Z = decltype(batch)::value;
                float t[Z][RPW];
#pragma unroll
                for (int u = 0; u < Z; ++u)
#pragma unroll
                    for (int rr = 0; rr < RPW; ++rr)
                        t[u][rr] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(pres, lane4, ((z0 + u) * NACC + wave * RPW + rr) * 256, 16));
#pragma unroll
                for (int u = 0; u < Z; ++u)
#pragma unroll
                    for (int rr = 0; rr < RPW; ++rr) v[rr] += t[u][rr];
            };
            constexpr int ZB = RPW <= 4 ? 8 : (RPW <= 16 ? 4 : 1);  // the largest batch the registers have room for
            int z0 = 0;
            for (; z0 + ZB <= nsplits; z0 += ZB) add_batch(z0, std::integral_constant<int, ZB>{});
            if (ZB > 4 && nsplits - z0 >= 4) {
                add_batch(z0, std::integral_constant<int, 4>{});
                z0 += 4;
            }
            if (ZB > 2 && nsplits - z0 >= 2) {
                add_batch(z0, std::integral_constant<int, 2>{});
                z0 += 2;
            }
            if (ZB > 1 && nsplits - z0 >= 1) add_batch(z0, std::integral_constant<int, 1>{});
            epilogue_all(v);
            if (first_thread()) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

#ifdef PAELLA_CONV_TIMELINE
    TL_STAMP(6);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    TL_STAMP(7);
    {
        const unsigned widx = bid * KW + (unsigned)wave;
        if (lane == 0 && g_tl_buf && widx < g_tl_cap) {
#pragma unroll
            for (int i = 0; i < 16; ++i) g_tl_buf[(size_t)widx * 16 + i] = tl[i];
        }
    }
#endif
    // End hook without a barrier: every wave waits for its own write-through stores, then counts itself in LDS; the wave that
    // completes the count reports the workgroup, the others leave the compute unit at once instead of waiting for the report's
    // round trip to the counter in memory (the wave slots they hold are what other workgroups are waiting for).
    if (p.notifier) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        bool last = true;
        if (KW > 1) {
            unsigned before = 0;
            if (lane == 0) before = __hip_atomic_fetch_add(&waves_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            last = __builtin_amdgcn_readfirstlane(before) == (unsigned)KW - 1;
        }
        if (last && lane == 0) p.notifier->end_from_one_lane(p.job_id & ~PAELLA_JOB_ID_FLAGS, (p.job_id & PAELLA_JOB_ID_TIME_BLOCKS) != 0, hook_blocks);
    }
}

// The second launch bound is waves per SIMD: eight is what the eight-wave workgroups of the small tile are planned for (four
// workgroups per compute unit), and the bound keeps the scalar registers within 96 as well -- a wave that takes more than 100
// of a SIMD's 800 leaves room for seven (three workgroups per compute unit).
template <int MI, int NI, int KW, bool TAP_MAJOR, int DEPTH = 0>
__global__ __launch_bounds__(64 * KW, (MI * NI == 1 && KW == 8 && DEPTH == 0) ? 8 : 1) void conv_mfma_kernel(ConvArgs args) {
    // The arguments are read through an index the compiler cannot see through (always 0), as the grouped kernel reads its
    // member's: a field is then fetched from the argument block where it is used instead of being held in a scalar register
    // from the first instruction to the epilogue (106 scalar registers and seven waves per SIMD otherwise, or 57 spills).
    int idx = 0;
    asm volatile("" : "+s"(idx));
    const ConvArgs& p = (&args)[idx];
    if (TAP_MAJOR && p.pointwise) conv_tile<MI, NI, KW, TAP_MAJOR, kPreNone, DEPTH, TAP_MAJOR>(p, blockIdx.x);
    else conv_tile<MI, NI, KW, TAP_MAJOR, kPreNone, DEPTH>(p, blockIdx.x);
}

// A conv that applies a per-channel transform to its input on the way (smallest tile, tap-major order).
struct ConvPreArgs {
    ConvArgs conv;
    PreOp pre;
};

template <int KW>
__device__ __forceinline__ void conv_pre_tile(const ConvPreArgs& a, unsigned bid) {
    const bool bounded = a.pre.lo > -__builtin_inff();
    if (a.conv.pointwise) {
        if (bounded) conv_tile<1, 1, KW, true, kPreBounded, 0, true>(a.conv, bid, a.pre);
        else conv_tile<1, 1, KW, true, kPreUnbounded, 0, true>(a.conv, bid, a.pre);
    } else {
        if (bounded) conv_tile<1, 1, KW, true, kPreBounded>(a.conv, bid, a.pre);
        else conv_tile<1, 1, KW, true, kPreUnbounded>(a.conv, bid, a.pre);
    }
}

template <int KW>
__global__ __launch_bounds__(64 * KW, KW == 8 ? 8 : 1) void conv_mfma_pre_kernel(ConvPreArgs args) {
    int idx = 0;  // see conv_mfma_kernel
    asm volatile("" : "+s"(idx));
    const ConvPreArgs& a = (&args)[idx];
    conv_pre_tile<KW>(a, blockIdx.x);
}

// The same for up to kPackMax such convs of different requests in one launch (launch packing).
struct ConvPreGroupArgs {
    unsigned start[PAELLA_CONV_PACK_MAX];  // first workgroup id of each problem; 0xFFFFFFFF for unused entries
    ConvPreArgs m[PAELLA_CONV_PACK_MAX];   // only the used entries are written to the argument ring
};

template <int KW>
__global__ __launch_bounds__(64 * KW, KW == 8 ? 8 : 1) void conv_mfma_pre_group_kernel(ConvPreGroupArgs g) {
    // The member's first workgroup id is carried along with its number: looked up afterwards, it is one more trip to the argument
    // block before the member's own arguments can be requested.
    int idx = 0;
    unsigned first = g.start[0];
#pragma unroll
    for (int i = 1; i < PAELLA_CONV_PACK_MAX; ++i)
        if (blockIdx.x >= g.start[i]) {
            idx = i;
            first = g.start[i];
        }
    conv_pre_tile<KW>(g.m[idx], blockIdx.x - first);
}

// Up to four independent convs in one launch: layers whose own grids would leave most of the 256 CUs idle (the 1x1
// projection beside a residual block's first 3x3, the parallel branches of an inception module) share a grid, one
// problem's workgroups after the other's.  All use the smallest tile and the same wave count; the hooks see one
// kernel of as many workgroups as the problems have together.  A workgroup finds its problem by its id and reads
// that problem's arguments (an index into the argument block, the same for the whole workgroup).
constexpr int kMaxGroup = PAELLA_CONV_GROUP_MAX;  // members of one call (one request's independent convs)
constexpr int kPackMax = PAELLA_CONV_PACK_MAX;    // members of one launch (the kernels of several requests packed together)

// A member may also be a pooling operator (an inception module starts with three 1x1 convs and a 3x3 pool that all read
// the module's input): its workgroups, one output element per thread with this kernel's workgroup size, come after all the
// convs' (they are the shortest).
// ... or a dense layer, one wave per output row (launches that carry the same stage of several small models' requests).
union GroupMember {
    ConvArgs conv;
    paella::PoolArgs pool;
    paella::DenseArgs dense;
    __host__ __device__ GroupMember() {}
};

enum MemberKind : unsigned { kMemberConv = 0, kMemberPool = 1, kMemberDense = 2 };

struct ConvGroupArgs {
    unsigned start[kPackMax];  // first workgroup id of each member; 0xFFFFFFFF for unused entries
    unsigned kinds;            // two bits per member: MemberKind
    unsigned reserved;
    GroupMember m[kPackMax];   // only the used entries are written to the argument ring
};

template <int KW, bool TAP_MAJOR>
__global__ __launch_bounds__(64 * KW, KW == 8 ? 8 : 1) void conv_mfma_group_kernel(ConvGroupArgs g) {
    int idx = 0;
    unsigned first = g.start[0];  // carried along: see conv_mfma_pre_group_kernel
#pragma unroll
    for (int i = 1; i < kPackMax; ++i)
        if (blockIdx.x >= g.start[i]) {
            idx = i;
            first = g.start[i];
        }
    const unsigned bid = blockIdx.x - first;
    const unsigned kind = (g.kinds >> (2 * idx)) & 3u;
    if (kind == kMemberPool) {
        const paella::PoolArgs& p = g.m[idx].pool;
        const unsigned blocks = p.hook_blocks ? p.hook_blocks : gridDim.x;
        paella::hook_entry(p.notifier, p.job_id, blocks);
        paella::pool_element(p, (int)(bid * (64 * KW) + threadIdx.x));
        paella::hook_exit(p.notifier, p.job_id, blocks);
        return;
    }
    if (kind == kMemberDense) {
        const paella::DenseArgs& d = g.m[idx].dense;
        const unsigned blocks = d.hook_blocks ? d.hook_blocks : gridDim.x;
        paella::hook_entry(d.notifier, d.job_id, blocks);
        paella::dense_row(d, (int)(bid * KW + (threadIdx.x >> 6)), (int)(threadIdx.x & 63));
        paella::hook_exit(d.notifier, d.job_id, blocks);
        return;
    }
    if (TAP_MAJOR && g.m[idx].conv.pointwise) conv_tile<1, 1, KW, TAP_MAJOR, false, 0, TAP_MAJOR>(g.m[idx].conv, bid);
    else conv_tile<1, 1, KW, TAP_MAJOR>(g.m[idx].conv, bid);
}

constexpr int kMaxGroupWithPool = 3;  // convs of one call that also carries a pooling operator

// ---------------------------------------------------------------------------------------------------
// Depthwise conv (groups == C == K): HBM-bound, one thread per output pixel, taps from L1/L2.

struct DwArgs {
    const float* x;
    const float* w;  // [C][R][S]
    const float* bias;
    const float* residual;
    const float* slope;
    float* y;
    int C, H, W, P, Q, R, S;
    int sh, sw, ph, pw, dh, dw;
    int act;
    float lo, hi;
    uint32_t job_id;
    llis::job::FinishedBlockNotifier* notifier;
    // 3 x 3 filters whose sizes the host has checked (fast = 1): output column and row by multiply-high, operands through buffer
    // descriptors with 32-bit offsets
    FastDiv div_q, div_p;
    int fast;
    unsigned x_bytes, out_bytes;
};

// All taps of one output element.  With the filter size known the loads of a window leave back to back (a tap outside the
// image reads element 0 of the channel and is replaced by zero afterwards) instead of one dependent trip to memory per tap;
// the sum runs in the same tap order either way, and a skipped tap and an added zero give the same bits.
template <int R, int S>
__device__ __forceinline__ float dw_window(const DwArgs& p, const float* xc, const float* wc, float acc, int h0, int w0) {
    float v[R * S], wt[R * S];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int h = h0 + r * p.dh, w = w0 + s * p.dw;
            const bool ok = (unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W;
            const float x = xc[ok ? h * p.W + w : 0];
            v[r * S + s] = ok ? x : 0.f;
            wt[r * S + s] = wc[r * S + s];
        }
#pragma unroll
    for (int t = 0; t < R * S; ++t) acc = fmaf(v[t], wt[t], acc);
    return acc;
}

// One output element of a depthwise conv.
__device__ __forceinline__ void dw_element(const DwArgs& p, int idx, int PQ) {
    const int c = idx / PQ;
    const int pix = idx - c * PQ;
    const int ho = pix / p.Q;
    const int wo = pix - ho * p.Q;
    const float* xc = p.x + (size_t)c * p.H * p.W;
    const float* wc = p.w + (size_t)c * p.R * p.S;
    float acc = p.bias ? p.bias[c] : 0.f;
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    if (p.R == 3 && p.S == 3) {
        acc = dw_window<3, 3>(p, xc, wc, acc, h0, w0);
    } else {
        for (int r = 0; r < p.R; ++r) {
            const int h = h0 + r * p.dh;
            if ((unsigned)h >= (unsigned)p.H) continue;
            for (int s = 0; s < p.S; ++s) {
                const int w = w0 + s * p.dw;
                if ((unsigned)w >= (unsigned)p.W) continue;
                acc = fmaf(xc[(size_t)h * p.W + w], wc[r * p.S + s], acc);
            }
        }
    }
    const size_t o = (size_t)idx;
    if (p.residual) acc += p.residual[o];
    const float sl = (p.act == PAELLA_ACT_PRELU) ? p.slope[c] : 0.f;
    store_out(p.y + o, apply_act(acc, p.act, sl, p.lo, p.hi));
}

// A thread computes kDwPerThread output elements, a whole grid apart from each other (neighbouring threads still touch
// neighbouring elements), when the launch was planned that way (grid * 256 < elements): a quarter of the workgroups for the
// large layers, whose kernels are bound by latency and not by the arithmetic, and with them a quarter of the end messages
// the serving thread has to read (MobileNetV2: 133 of its 254 messages per request came from seven depthwise layers).
constexpr int kDwPerThread = 4;
constexpr int kDwWideFrom = 65536;  // elements from which a thread takes several

// K output elements of a 3 x 3 depthwise conv, a grid stride apart, with every operand of all K requested before the first
// multiply.  Addresses are 32-bit offsets into buffer descriptors: a tap outside the image gets an offset out of range and
// reads as zero, a thread past the last element computes the last one again and has its store dropped -- no branch and no
// 64-bit address per load (the plain form above spends some 190 vector instructions per element, most of them on addresses,
// and waits for memory once per element).  Same taps in the same order: the same bits as dw_element.
template <int K>
__device__ __forceinline__ void dw_batch3x3(const DwArgs& p, const int idx, const int stride, const int total) {
    // the input through a descriptor that starts (pad_h * W + pad_w) elements in front of it, so that a lane's offset -- that of
    // input element (ho * stride_h, wo * stride_w) of its channel -- is never negative; a tap's share is wave-uniform
    const unsigned pad_off = (unsigned)(p.ph * p.W + p.pw) * 4u;
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)(reinterpret_cast<const char*>(p.x) - pad_off), 0, p.x_bytes + pad_off, 0x00027000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, (unsigned)p.C * 36u, 0x00027000);
    const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc((void*)p.bias, 0, p.bias ? (unsigned)p.C * 4u : 0u, 0x00027000);
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc((void*)p.residual, 0, p.residual ? p.out_bytes : 0u, 0x00027000);
    const __amdgpu_buffer_rsrc_t sr = __builtin_amdgcn_make_buffer_rsrc((void*)p.slope, 0, p.act == PAELLA_ACT_PRELU ? (unsigned)p.C * 4u : 0u, 0x00027000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc((void*)p.y, 0, p.out_bytes, 0x00027000);
    int tap_soff[9];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int t = 0; t < 3; ++t) tap_soff[r * 3 + t] = (r * p.dh * p.W + t * p.dw) * 4;
    float v[K][9], wt[K][9], acc[K], res[K], sl[K];
    int out_off[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int i = idx + k * stride;
        const bool live = i < total;
        const int e = live ? i : total - 1;
        const int row = (int)quot_fast((unsigned)e, p.div_q);  // over (channel, output row)
        // every factor below is under 2^23 (checked by the host): 24-bit multiplies, a quarter of the passes of a 32-bit one
        const int wo = e - __mul24(row, p.Q);
        const int c = (int)quot_fast((unsigned)row, p.div_p);
        const int ho = row - __mul24(c, p.P);
        const int hs = __mul24(ho, p.sh), ws = __mul24(wo, p.sw);
        const int h0 = hs - p.ph, w0 = ws - p.pw;
        const int base = (__mul24(__mul24(c, p.H) + hs, p.W) + ws) * 4;
        // a row or a column outside the image sets the offset's top bit: beyond any length, the tap reads as zero (three-operand
        // `or` per tap; flags combined as booleans cost five vector instructions per tap)
        int row_bad[3], col_bad[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            row_bad[r] = (unsigned)(h0 + r * p.dh) < (unsigned)p.H ? 0 : (int)0x80000000u;
            col_bad[r] = (unsigned)(w0 + r * p.dw) < (unsigned)p.W ? 0 : (int)0x80000000u;
        }
#pragma unroll
        for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int t = 0; t < 3; ++t)
                v[k][r * 3 + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, base | row_bad[r] | col_bad[t], tap_soff[r * 3 + t], 0));
        const int woff = __mul24(c, 36);
#pragma unroll
        for (int t = 0; t < 9; ++t) wt[k][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(wr, woff, t * 4, 0));
        acc[k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, c * 4, 0, 0));
        out_off[k] = live ? e * 4 : -1;
        res[k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rr, out_off[k], 0, 0));
        sl[k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sr, c * 4, 0, 0));  // length zero unless PReLU
    }
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int t = 0; t < 9; ++t) acc[k] = fmaf(v[k][t], wt[k][t], acc[k]);
    if (p.residual) {  // (not added as a zero: -0 + 0 is +0)
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] += res[k];
    }
    const int act = p.act;  // one scalar branch per kind of activation around all K elements
    if (act == PAELLA_ACT_RELU) {
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = fmaxf(acc[k], 0.f);
    } else if (act == PAELLA_ACT_RELU6) {
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = fminf(fmaxf(acc[k], 0.f), 6.f);
    } else if (act == PAELLA_ACT_PRELU) {
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = acc[k] > 0.f ? acc[k] : acc[k] * sl[k];
    } else if (act == PAELLA_ACT_CLIP) {
        const float lo = p.lo, hi = p.hi;
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = fminf(fmaxf(acc[k], lo), hi);
    }
#pragma unroll
    for (int k = 0; k < K; ++k)  // write-through (sc1), like store_out
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, acc[k]), yr, out_off[k], 0, 16);
}

// One workgroup's share of a depthwise conv of `grid` workgroups.
__device__ __forceinline__ void dw_block(const DwArgs& p, const unsigned bid, const unsigned grid) {
    const int PQ = p.P * p.Q;
    const int total = p.C * PQ;
    const int stride = (int)grid * 256;
    int idx = (int)bid * 256 + threadIdx.x;  // over (channel, pixel): small feature maps still fill their workgroups
    if (p.fast) {
        if (stride >= total) dw_batch3x3<1>(p, idx, stride, total);
        else dw_batch3x3<kDwPerThread>(p, idx, stride, total);
        return;
    }
    if (stride >= total) {
        if (idx < total) dw_element(p, idx, PQ);
    } else {
#pragma unroll
        for (int k = 0; k < kDwPerThread; ++k, idx += stride)
            if (idx < total) dw_element(p, idx, PQ);
    }
}

__global__ __launch_bounds__(256) void dwconv_kernel(DwArgs p) {
    paella::hook_entry(p.notifier, p.job_id);
    dw_block(p, blockIdx.x, gridDim.x);
    paella::hook_exit(p.notifier, p.job_id);
}

// The same for up to PAELLA_CONV_PACK_MAX depthwise convs of different requests in one launch (launch packing): a model of
// many short kernels is bound by how many launches the four queues start per second, and its depthwise layers are a third
// of them.  A member's workgroups behave exactly as in a launch of their own (same elements per thread, same messages).
struct DwGroupArgs {
    unsigned start[PAELLA_CONV_PACK_MAX];  // first workgroup id of each member; 0xFFFFFFFF for unused entries
    unsigned grids[PAELLA_CONV_PACK_MAX];  // workgroups of each member
    DwArgs m[PAELLA_CONV_PACK_MAX];        // only the used entries are written to the argument ring
};

__global__ __launch_bounds__(256) void dwconv_group_kernel(DwGroupArgs g) {
    int member = 0;
    unsigned first = g.start[0], grid = g.grids[0];  // carried along: see conv_mfma_pre_group_kernel
#pragma unroll
    for (int i = 1; i < PAELLA_CONV_PACK_MAX; ++i)
        if (blockIdx.x >= g.start[i]) {
            member = i;
            first = g.start[i];
            grid = g.grids[i];
        }
    const DwArgs& p = g.m[member];
    const unsigned bid = blockIdx.x - first;
    paella::hook_entry(p.notifier, p.job_id, grid);
    dw_block(p, bid, grid);
    paella::hook_exit(p.notifier, p.job_id, grid);
}

typedef void (*ConvKernel)(ConvArgs);

template <int MI, int NI, bool TM>
ConvKernel pick_kw(int kw) {
    switch (kw) {
        case 1: return conv_mfma_kernel<MI, NI, 1, TM>;
        case 2: return conv_mfma_kernel<MI, NI, 2, TM>;
        case 4: return conv_mfma_kernel<MI, NI, 4, TM>;
        case 8: return conv_mfma_kernel<MI, NI, 8, TM>;
        default: return nullptr;
    }
}

template <bool TM>
ConvKernel pick_tile(int mi, int ni, int kw) {
    if (mi == 1 && ni == 1) return pick_kw<1, 1, TM>(kw);
    if (mi == 1 && ni == 2) return pick_kw<1, 2, TM>(kw);
    if (mi == 2 && ni == 1) return pick_kw<2, 1, TM>(kw);
    if (mi == 2 && ni == 2) return pick_kw<2, 2, TM>(kw);
    return nullptr;
}

// Variants of the 32 x 32 tap-major kernel with fewer waves per tile and more chunks of operands in flight per wave.
template <int KW>
ConvKernel pick_depth(int depth) {
    switch (depth) {
        case 3: return conv_mfma_kernel<1, 1, KW, true, 3>;
        case 4: return conv_mfma_kernel<1, 1, KW, true, 4>;
        case 6: return conv_mfma_kernel<1, 1, KW, true, 6>;
        case 8: return conv_mfma_kernel<1, 1, KW, true, 8>;
        case 12: return conv_mfma_kernel<1, 1, KW, true, 12>;
        default: return nullptr;
    }
}

ConvKernel pick_deep_kernel(int kw, int depth) {
    switch (kw) {
        case 1: return pick_depth<1>(depth);
        case 2: return pick_depth<2>(depth);
        case 4: return pick_depth<4>(depth);
        case 8: return pick_depth<8>(depth);
        default: return nullptr;
    }
}

ConvKernel pick_kernel(int mi, int ni, int kw, int k_order = 0, int depth = 0) {
    if (depth) return (mi == 1 && ni == 1 && k_order) ? pick_deep_kernel(kw, depth) : nullptr;
    return k_order ? pick_tile<true>(mi, ni, kw) : pick_tile<false>(mi, ni, kw);
}

constexpr size_t kMaxSplitTiles = 16384;  // counters at the head of a split-k workspace

int conv_out(int in, int k, int stride, int pad, int dil) { return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1; }

int round_up(int v, int m) { return (v + m - 1) / m * m; }

FastDiv fast_div(unsigned d) {
    if (d <= 1) return FastDiv{0u, 0xFFFFFFFFu};
    return FastDiv{(unsigned)((((uint64_t)1) << 32) / d + 1), 0u};
}

}  // namespace

extern "C" int paella_conv2d_plan(const paella_conv_desc* d, int has_residual, int tile_hint, paella_conv_plan* plan) {
    if (!d || !plan) return PAELLA_EINVAL;
    if (d->C <= 0 || d->H <= 0 || d->W <= 0 || d->K <= 0 || d->R <= 0 || d->S <= 0 || d->stride_h <= 0 ||
        d->stride_w <= 0 || d->pad_h < 0 || d->pad_w < 0 || d->dil_h <= 0 || d->dil_w <= 0 || d->groups <= 0)
        return PAELLA_EINVAL;
    if (d->act < PAELLA_ACT_NONE || d->act > PAELLA_ACT_CLIP) return PAELLA_EINVAL;
    const int P = conv_out(d->H, d->R, d->stride_h, d->pad_h, d->dil_h);
    const int Q = conv_out(d->W, d->S, d->stride_w, d->pad_w, d->dil_w);
    if (P <= 0 || Q <= 0) return PAELLA_EINVAL;
    // Offsets are 32-bit byte offsets and (r*dil, s*dil) are packed into 16 bits each.
    if ((double)d->C * d->H * d->W * 4 >= 2147483648.0 || (d->R - 1) * d->dil_h >= 0x7000 || (d->S - 1) * d->dil_w >= 0x7000)
        return PAELLA_ENOSUP;
    // ... and so are the output's (a lane's offset within its tile's channels is held against the tensor's length in bytes)
    if ((double)(d->K + 64) * P * Q * 4 >= 2147483648.0) return PAELLA_ENOSUP;

    std::memset(plan, 0, sizeof(*plan));
    plan->d = *d;
    plan->P = P;
    plan->Q = Q;
    const int PQ = P * Q;
    const int cg = d->C / d->groups;
    plan->flops = 2.0 * d->K * cg * d->R * d->S * PQ;
    plan->bytes = 4.0 * ((double)d->C * d->H * d->W + (double)d->K * cg * d->R * d->S + d->K + (double)d->K * PQ * (has_residual ? 2 : 1));

    if (d->groups == 1) {
        plan->kind = 0;
        const int kdim = d->C * d->R * d->S;
        const int k_pad = round_up(kdim, 8);
        const int nchunks = k_pad / 8;
        int mi, ni, kw;
        auto tiles = [&](int a, int b) { return ((d->K + 32 * a - 1) / (32 * a)) * ((PQ + 32 * b - 1) / (32 * b)); };
        if (tile_hint > 0) {
            mi = (tile_hint >> 8) & 0xF;
            ni = (tile_hint >> 4) & 0xF;
            kw = 1 << (tile_hint & 0xF);
            if (!pick_kernel(mi, ni, kw)) return PAELLA_EINVAL;
            plan->depth = (tile_hint >> 16) & 0xF;
            if (plan->depth && !pick_kernel(mi, ni, kw, d->C % 8 == 0 ? 1 : 0, plan->depth)) return PAELLA_EINVAL;
        } else {
            // The 32 x 32 tile unless it would make thousands of workgroups: measured on the layers of the model zoo
            // (one launch at a time) it is the fastest or within 3 % of the fastest everywhere, and up to twice as fast
            // as the larger tiles on layers with few channels (stems, first pointwise layers).  Waves per workgroup:
            // the power of two that covers the chunks of the reduction, between 2 and 8 -- a wave with a single chunk
            // still beats fewer waves with two.
            if (tiles(1, 1) <= 2048) { mi = 1; ni = 1; }
            else if (tiles(1, 2) <= 2048 || d->K <= 32) { mi = 1; ni = 2; }
            else { mi = 2; ni = 2; }
            // The same holds with four passes in flight, where throughput rather than latency might have favoured operand
            // reuse (ResNet-18, thousand passes per second, four queues / one): 32 x 32 everywhere 15.8 / 7.0; 64 x 32 where
            // K is a multiple of 64: 12.1 / 4.9, only from K = 256: 13.2 / 5.6; 32 x 64 on the 56 x 56 layers: 14.4 / 6.4.
            // (at most 4 where the reduction goes through the offset table -- stems: 7.8 against 7.9 us, 4.4 against 4.7)
            static const int kw_cap = [] { const char* e = std::getenv("PAELLA_CONV_KW_MAX"); const int v = e ? std::atoi(e) : 8; return v == 1 || v == 2 || v == 4 ? v : 8; }();
            const int kw_max = std::min(d->C % 8 == 0 ? 8 : 4, kw_cap);
            kw = 2;
            while (kw < kw_max && kw < nchunks) kw <<= 1;
            // (Served, too: at least two or three chunks per wave, i.e. four waves for a 64-channel pointwise layer, gives ResNet-50
            // 7.10 against 7.43 thousand requests/s and MobileNetV2, DenseNet-121 and SqueezeNet 1 % less each.)
            // (Four waves per tile for layers of 640 or 1024 tiles and more, where the device is filled several times over either
            // way and half the waves would do half the per-wave scalar work: +0.5 % with the device full, -1.4 % served.)
        }
        // Grid-level split of the reduction: layers with few output tiles (small feature maps) would otherwise
        // occupy a fraction of the 256 CUs.  Aim at about one workgroup per CU and keep a minimum of chunks per wave (below).
        // Measured on ResNet-18 with four passes in flight / one pass alone (thousand passes per second), by the cap
        // on workgroups and the waves per workgroup: 288 x 8: 15.2 / 6.9;
        // 288 x 4: 14.5 / 6.1; 144 x 8: 13.7 / 6.1; 144 x 4: 11.9 / 5.1; 576 x 8: 13.8 / 6.0.
        const int n_tiles = tiles(mi, ni);
        int splits = 1;
        if (tile_hint > 0) {
            splits = 1 << ((tile_hint >> 12) & 0xF);
        } else {
            const int cap = 288;
            // How far the split goes is a trade between a kernel's latency (more, smaller workgroups) and the fixed cost of a
            // workgroup and of the exchange of partial tiles (fewer, larger ones).  Layers under 16 MFLOP go down to 2 chunks per
            // wave, the others kept 6 at first.  Served by full3 at saturation, median of three runs, requests/s against the earlier rule
            // (2 chunks for layers of at most 32 tiles, 4 otherwise): Inception-v3 4310 -> 4630, ResNet-50 5490 -> 5605,
            // GoogLeNet 9520 -> 9500, MobileNetV2 8390 -> 8240, DenseNet-121 3650 -> 3540 (its 25-50 MFLOP pointwise layers on
            // 14 x 14 maps are a pure chain and would rather be split), small CNN : Inception-v3 = 9 : 1 35.9 -> 37.1 thousand;
            // four passes in flight without scheduler: Inception-v3 4.81 -> 5.00 thousand passes/s; one launch at a time 9.09 ->
            // 9.20 us.  Thresholds of 32 and 64 MFLOP gave Inception-v3 4617 and 4443; 5 or 8 chunks instead of 6: 4552, 4588.
            // With launches of several requests packed together (paella_pack_*) the parallelism that splits provided comes from
            // the other requests, and the same measurement (one box, packing on) moved the larger layers to 9 chunks per wave:
            // 6 / 8 / 9 / 10 / 12 chunks: Inception-v3 5036 / 5238 / 5286 / 5306 / 5323, ResNet-50 6381 / 6325 / 6438 / 6447 / 6430,
            // DenseNet-121 5173 / 5159 / 5139 / 5043 / 5013 requests/s, the 9 : 1 mix 43.9 / 44.9 / 44.6 / 44.8 / 44.9 thousand.
            // Once more with the split path cheapened (uniform bookkeeping, exact batches): 4 / 6 / 9 / 12 chunks: Inception-v3 served
            // with 32 requests outstanding 5.58 / 6.18 / 6.58 / 6.73 thousand, with 16: 5.39 / 5.79 / 6.00 / 6.02, ResNet-50 7.21 / 7.43 /
            // 7.45 / 7.38, the 9 : 1 mix 49.5 / 51.6 / 53.5 / 53.4 thousand, one launch at a time 7.9 / 7.9 / 7.91 / 8.05 us: 9 stays.
            const int min_chunks = plan->flops < 16e6 ? 2 : 9;
            while (splits < 16 && n_tiles * splits * 2 <= cap && nchunks / (splits * 2 * kw) >= min_chunks) splits *= 2;
        }
        int chunks_per_split = (nchunks + splits - 1) / splits;
        splits = (nchunks + chunks_per_split - 1) / chunks_per_split;  // no empty split
        plan->mi = mi;
        plan->ni = ni;
        plan->kw = kw;
        plan->splits = splits;
        plan->m_pad = round_up(d->K, 32 * mi);
        plan->k_pad = k_pad;
        // Reduction order: (r, s, c) when whole chunks of 8 share a filter tap, else (c, r, s) with the offset table.
        plan->k_order = d->C % 8 == 0 ? 1 : 0;
        // Stride 2 across a 3-wide filter: the two columns that read pixels (2 q, 2 q + 1) are paired (see the kernel's operand
        // fetch) when both lie inside the image for every output column, 2 Q <= W.
        {
            static const bool pairing = [] { const char* e = std::getenv("PAELLA_CONV_PAIR_TAPS"); return !e || std::atoi(e) != 0; }();
            plan->pair_taps = (pairing && plan->k_order && mi == 1 && ni == 1 && d->S == 3 && d->stride_w == 2 && d->dil_w == 1 && d->pad_w <= 1 && 2 * Q <= d->W)
                                  ? 1 + d->pad_w : 0;
        }
        // Which workgroups share an XCD.  Weights outweigh the input: those that read one slab of weights; else neighbouring pixels.
        plan->wg_order = (double)d->K * d->C * d->R * d->S > (double)d->C * d->H * d->W ? 1 : 0;
        plan->fast_div = 1;
        plan->blob_bytes = (size_t)(k_pad / 4) * plan->m_pad * sizeof(float4);
        if (plan->blob_bytes >= ((size_t)1 << 31)) return PAELLA_ENOSUP;  // weights are addressed with 32-bit byte offsets
        // Workspace = fixed-size counter area (so that stages of one request, which share the workspace, never
        // see each other's partial sums where they expect zeroed counters) followed by the partial tiles.
        if (splits > 1 && n_tiles > kMaxSplitTiles) return PAELLA_ENOSUP;
        plan->workspace_bytes = splits > 1 ? kMaxSplitTiles * sizeof(unsigned) + (size_t)n_tiles * splits * (mi * ni * 16 * 64) * sizeof(float) : 0;
        plan->dims.grid = (unsigned)(n_tiles * splits);
        plan->dims.block = 64u * kw;
        {
            const unsigned red_bytes = kw > 1 ? (unsigned)(kw * mi * ni * 16 * 64 * sizeof(float)) : 0u;
            const unsigned tab_bytes = plan->k_order ? 0u : (unsigned)(chunks_per_split * 8 * sizeof(int2));
            plan->dims.lds_bytes = red_bytes > tab_bytes ? red_bytes : tab_bytes;
            if (plan->dims.lds_bytes > 160 * 1024) return PAELLA_ENOSUP;  // table does not fit the CU's LDS
        }
        plan->dims.vgprs = 128;
        return 0;
    }
    if (d->groups == d->C && d->K == d->C) {
        plan->kind = 1;
        plan->blob_bytes = (size_t)d->C * d->R * d->S * sizeof(float);
        if ((double)d->C * PQ >= 2147483648.0) return PAELLA_ENOSUP;  // output elements are indexed with 32 bits
        {
            const size_t elements = (size_t)d->C * PQ;
            const size_t per_group = elements >= (size_t)kDwWideFrom ? 256u * (size_t)kDwPerThread : 256u;
            plan->dims.grid = (unsigned)((elements + per_group - 1) / per_group);
        }
        plan->dims.block = 256;
        plan->dims.lds_bytes = 0;
        plan->dims.vgprs = 32;
        return 0;
    }
    return PAELLA_ENOSUP;
}

extern "C" int paella_conv2d_pack(const paella_conv_plan* plan, const float* w, void* blob_host) {
    if (!plan || !w || !blob_host) return PAELLA_EINVAL;
    const paella_conv_desc& d = plan->d;
    if (plan->kind == 1) {
        std::memcpy(blob_host, w, plan->blob_bytes);
        return 0;
    }
    const int kdim = d.C * d.R * d.S;
    float* wp = reinterpret_cast<float*>(blob_host);
    std::memset(wp, 0, (size_t)(plan->k_pad / 4) * plan->m_pad * sizeof(float4));
    const int RS = d.R * d.S;
    for (int m = 0; m < d.K; ++m)
        for (int k = 0; k < kdim; ++k) {  // k indexes the source in (c, r, s) order
            int kp = plan->k_order ? (k % RS) * d.C + k / RS : k;  // position in the kernel's reduction order
            if (plan->pair_taps) {
                // per filter row: the unpaired column's C values, then the pair's 2 C values as chunks of (column 0 | column 1) x
                // four channels
                const int c = k / RS, r = (k % RS) / d.S, sx = k % d.S, s0 = plan->pair_taps - 1;
                if (sx == 2 - 2 * s0) kp = r * 3 * d.C + c;
                else kp = r * 3 * d.C + d.C + (c / 4) * 8 + (sx - s0) * 4 + (c % 4);
            }
            wp[((size_t)(kp / 4) * plan->m_pad + m) * 4 + (kp % 4)] = w[(size_t)m * kdim + k];
        }
    return 0;
}

namespace {

// Kernel arguments of one MFMA conv (plan->kind == 0).
int fill_args(const paella_conv_plan* plan, const float* x, const void* blob_dev, const float* bias, const float* residual,
              const float* slope, float* y, void* workspace, uint32_t job_id, llis::job::FinishedBlockNotifier* nf, ConvArgs& a) {
    if (!plan || !x || !blob_dev || !y || plan->kind != 0) return PAELLA_EINVAL;
    const paella_conv_desc& d = plan->d;
    if (d.act == PAELLA_ACT_PRELU && !slope) return PAELLA_EINVAL;
    const int PQ = plan->P * plan->Q;
    a.x = x;
    a.wpk = reinterpret_cast<const float4*>(blob_dev);
    a.w_bytes = (unsigned)plan->blob_bytes;
    a.kdim = d.C * d.R * d.S; a.RS = d.R * d.S; a.S = d.S; a.dh = d.dil_h; a.dw = d.dil_w;
    a.CB = d.C / 8;
    a.bias = bias;
    a.residual = residual;
    a.slope = slope;
    a.y = y;
    a.H = d.H; a.W = d.W; a.Q = plan->Q; a.PQ = PQ;
    a.sh = d.stride_h; a.sw = d.stride_w; a.ph = d.pad_h; a.pw = d.pad_w;
    a.K = d.K; a.m_pad = plan->m_pad; a.nchunks = plan->k_pad / 8;
    a.splits = plan->splits;
    a.chunks_per_split = (a.nchunks + plan->splits - 1) / plan->splits;
    a.ws_partials = nullptr;
    a.ws_counters = nullptr;
    if (plan->splits > 1) {
        if (!workspace) return PAELLA_EINVAL;
        // counters first (they must be zero before the first launch; the kernel leaves them at zero)
        a.ws_counters = reinterpret_cast<unsigned*>(workspace);
        a.ws_partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kMaxSplitTiles * sizeof(unsigned));
    }
    a.x_bytes = (unsigned)((size_t)d.C * d.H * d.W * 4);
    a.act = d.act; a.lo = d.act_lo; a.hi = d.act_hi;
    a.job_id = job_id;
    a.hook_blocks = plan->dims.grid;  // a launch of its own: all of its workgroups (0 would make the kernel fetch the grid size itself)
    a.notifier = nf;
    a.n_tiles_n = (PQ + 32 * plan->ni - 1) / (32 * plan->ni);
    a.n_tiles_m = plan->m_pad / (32 * plan->mi);
    a.slab_major = plan->wg_order;
    // Divisions by multiply-high: every dividend of the kernel is below `most`, every divisor at most `widest`.
    const unsigned d_w = a.slab_major ? (unsigned)a.n_tiles_n : (unsigned)(a.n_tiles_m * a.splits);
    const unsigned d_cb = a.CB > 0 ? (unsigned)a.CB : 1u;  // unused when C is no multiple of 8
    a.div_w = fast_div(d_w);
    a.div_tm = fast_div((unsigned)a.n_tiles_m);
    a.div_q = fast_div((unsigned)plan->Q);
    a.div_cb = fast_div(d_cb);
    a.div_s = fast_div((unsigned)d.S);
    const uint64_t total = (uint64_t)a.n_tiles_n * a.n_tiles_m * a.splits;
    const uint64_t most = std::max<uint64_t>({total, (uint64_t)a.n_tiles_n * 32 * plan->ni, (uint64_t)a.nchunks + a.chunks_per_split});
    const uint64_t widest = std::max<uint64_t>({d_w, (uint64_t)a.n_tiles_m, (uint64_t)plan->Q, d_cb, (uint64_t)d.S});
    a.fast_div = (plan->fast_div && most * widest < ((uint64_t)1 << 32)) ? 1 : 0;
    // The reduction loop locates its chunks with the multiply-high alone (chunk by chunks per tap, tap by filter width).
    if (((uint64_t)a.nchunks + a.chunks_per_split + 64) * std::max<uint64_t>(d_cb, (uint64_t)d.S) >= ((uint64_t)1 << 32)) return PAELLA_ENOSUP;
    a.pointwise = plan->k_order && d.R == 1 && d.S == 1 && d.stride_h == 1 && d.stride_w == 1 && d.pad_h == 0 && d.pad_w == 0 ? 1 : 0;
    a.pair_s0 = plan->pair_taps - 1;
    return 0;
}

int allow_lds(const void* kern, unsigned lds_bytes) {
    if (lds_bytes <= 65536) return 0;
    return (int)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
}

// What the scheduler accounts for a launch of `fn`: the kernel's own register count and, on top of the dynamic LDS already
// in dims, its statically allocated LDS -- both read from the loaded code object (left as planned without a device).
void add_kernel_resources(const void* fn, paella_launch_dims* dims) {
    hipFuncAttributes attr;
    if (fn && hipFuncGetAttributes(&attr, fn) == hipSuccess && attr.numRegs > 0) {
        dims->vgprs = (unsigned)attr.numRegs;
        dims->lds_bytes += (unsigned)attr.sharedSizeBytes;
    } else {
        (void)hipGetLastError();
    }
}

typedef void (*ConvGroupKernel)(ConvGroupArgs);

ConvGroupKernel pick_group_kernel(int kw, int k_order) {
    switch (kw) {
        case 1: return k_order ? conv_mfma_group_kernel<1, true> : conv_mfma_group_kernel<1, false>;
        case 2: return k_order ? conv_mfma_group_kernel<2, true> : conv_mfma_group_kernel<2, false>;
        case 4: return k_order ? conv_mfma_group_kernel<4, true> : conv_mfma_group_kernel<4, false>;
        case 8: return k_order ? conv_mfma_group_kernel<8, true> : conv_mfma_group_kernel<8, false>;
        default: return nullptr;
    }
}

}  // namespace

extern "C" int paella_conv2d_group_dims(const paella_conv_plan* const* plans, int n, paella_launch_dims* dims) {
    if (!plans || n < 2 || n > kMaxGroup) return PAELLA_EINVAL;
    for (int i = 0; i < n; ++i) {
        if (!plans[i]) return PAELLA_EINVAL;
        const paella_conv_plan& p = *plans[i];
        if (p.kind != 0 || p.mi != 1 || p.ni != 1 || p.kw != plans[0]->kw || p.k_order != plans[0]->k_order) return PAELLA_ENOSUP;
    }
    if (dims) {
        dims->grid = 0;
        dims->lds_bytes = 0;
        for (int i = 0; i < n; ++i) {
            dims->grid += plans[i]->dims.grid;
            if (plans[i]->dims.lds_bytes > dims->lds_bytes) dims->lds_bytes = plans[i]->dims.lds_bytes;
        }
        dims->block = plans[0]->dims.block;
        dims->vgprs = plans[0]->dims.vgprs;
        add_kernel_resources(reinterpret_cast<const void*>(pick_group_kernel(plans[0]->kw, plans[0]->k_order)), dims);
    }
    return 0;
}

namespace {

// First workgroup id of the next conv of a grouped launch.  Workgroup ids are dealt round-robin over the eight XCDs, and
// conv_tile gives the ids of one XCD a contiguous run of the problem's work list (same weights or neighbouring pixels in one
// L2): that only holds for a problem whose first id is a multiple of eight.
unsigned align_start(unsigned next) { return (next + 7u) & ~7u; }

// One launch of the group kernel over the first n members of g (their start[] and kinds filled; the rest marked
// unused here).
int launch_group_args(ConvGroupArgs& g, int n, int kw, int k_order, unsigned grid, unsigned dyn_lds, void* stream) {
    for (int i = n; i < kPackMax; ++i) g.start[i] = 0xFFFFFFFFu;
    g.reserved = 0;
    ConvGroupKernel kern = pick_group_kernel(kw, k_order);
    if (!kern) return PAELLA_EINVAL;
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), dyn_lds)) return rc;
    paella::launch_used(kern, dim3(grid), dim3(64u * (unsigned)kw), dyn_lds, reinterpret_cast<hipStream_t>(stream),
                        offsetof(ConvGroupArgs, m) + (size_t)n * sizeof(GroupMember), g);
    return (int)hipGetLastError();
}

// ---- Launch packing ---------------------------------------------------------------------------------------------
// A hardware queue of this device runs one kernel at a time, and four queues is all that run side by side: a conv that
// fills a fifth of the machine still takes a queue for its whole latency.  With packing on (paella_pack_enable, per
// thread), conv launches on the 32 x 32 tile that are bound for an unordered direct-dispatch queue are held back and go
// out together, up to kPackMax problems in one grid of the group kernel, each with its own job id and notifier.  The
// holder (the serving thread) calls paella_pack_poll() from its loop: what is held goes out as soon as a queue of the
// shared set has nothing waiting, when a launch is full, or after kPackHoldNs at the latest.
struct PackItem {
    int n = 0;               // convs of one call (one job's stage)
    bool has_pool = false;   // ... and the pooling operator that goes with them
    unsigned grid = 0;       // their workgroups together: what the job's notifier counts
    unsigned dyn_lds = 0;
    ConvArgs args[kMaxGroup];
    unsigned grids[kMaxGroup];
    paella::PoolArgs pool;
    unsigned pool_grid = 0;
    int members() const { return n + (has_pool ? 1 : 0); }
};

struct PackList {
    std::vector<PackItem> items;
    int members = 0;
};

// A job's whole ordered launch sequence (a model of small kernels is one scheduler stage), recorded between
// paella_pack_sequence_begin and _end: the sequences of several requests of one model go out position by position, the
// k-th launches of all of them in one grid, on one queue with the barrier bit set.
struct SeqRecord {
    unsigned kind = kMemberConv;
    int kw = 4, k_order = 1;   // conv: the kernel variant; pool and dense ride in the <4, tap-major> variant, whose 256-thread
                               // workgroups make their grids what the stand-alone kernels' are (the scheduler counts on that)
    unsigned dyn_lds = 0;
    unsigned units = 0;        // conv: workgroups; pool: output elements; dense: output rows
    GroupMember m;
};

struct Sequence {
    std::vector<SeqRecord> recs;
};

struct SeqList {
    const void* key = nullptr;
    std::vector<Sequence> seqs;
};

struct PackState {
    bool enabled = false;
    int held = 0;                 // items and sequences over all lists
    uint64_t first_held_ns = 0;
    PackList lists[4][2];         // by log2(waves per workgroup) and reduction order
    struct DwItem {
        DwArgs a;
        unsigned grid;
    };
    std::vector<DwItem> dw_list;   // depthwise convs, packed among themselves
    std::vector<SeqList> seq_lists;
    struct PreItem {
        ConvPreArgs a;
        unsigned grid = 0, dyn_lds = 0;
    };
    std::vector<PreItem> pre_lists[4];  // convs with a fused input transform, by log2(waves per workgroup)
    const void* rec_key = nullptr;  // the sequence being recorded (paella::g_pack_recording says whether one is)
    void* rec_queue = nullptr;
    Sequence rec;
};

std::atomic<uint64_t> g_pack_launches{0}, g_pack_members{0};  // over all threads, for reports

thread_local PackState g_pack;
constexpr uint64_t kPackHoldNs = 30000;

uint64_t now_ns() {
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (uint64_t)ts.tv_sec * 1000000000ull + (uint64_t)ts.tv_nsec;
}

int kw_index(int kw) { return kw == 1 ? 0 : kw == 2 ? 1 : kw == 4 ? 2 : 3; }

// Holds the call back if packing applies to it.  Returns false when the caller must launch it itself.
// A depthwise conv bound for an unordered direct queue is held like a small-tile conv and packed with other requests' depthwise convs.
bool pack_hold_dw(const DwArgs& a, unsigned grid, void* stream) {
    if (paella::g_pack_recording || !g_pack.enabled || paella::timing_events().start != nullptr) return false;
    paella::DirectQueue* q = paella::direct_queue_lookup(stream);
    if (!q || paella::direct_queue_ordered(q)) return false;
    g_pack.dw_list.push_back(PackState::DwItem{a, grid});
    if (g_pack.held++ == 0) g_pack.first_held_ns = now_ns();
    return true;
}

int dw_send_all(bool only_full) {
    std::vector<PackState::DwItem>& list = g_pack.dw_list;
    int launches = 0;
    size_t done = 0;
    bool failed = false;
    while (done < list.size()) {
        const size_t left = list.size() - done;
        if (only_full && left < (size_t)kPackMax) break;
        const int n = (int)std::min<size_t>(left, (size_t)kPackMax);
        void* target = nullptr;
        int rc = paella_direct_queue_shared(&target) != 0 ? -1 : 0;
        if (rc != 0) {
        } else if (n == 1) {
            paella::launch(dwconv_kernel, dim3(list[done].grid), dim3(256), 0, reinterpret_cast<hipStream_t>(target), list[done].a);
            rc = (int)hipGetLastError();
        } else {
            DwGroupArgs g;
            unsigned grid = 0;
            for (int i = 0; i < n; ++i) {
                g.m[i] = list[done + (size_t)i].a;
                g.start[i] = grid;
                g.grids[i] = list[done + (size_t)i].grid;
                grid += g.grids[i];
            }
            for (int i = n; i < kPackMax; ++i) {
                g.start[i] = 0xFFFFFFFFu;
                g.grids[i] = 0;
            }
            paella::launch_used(dwconv_group_kernel, dim3(grid), dim3(256), 0, reinterpret_cast<hipStream_t>(target),
                                offsetof(DwGroupArgs, m) + (size_t)n * sizeof(DwArgs), g);
            rc = (int)hipGetLastError();
        }
        if (rc != 0) {
            failed = true;
            break;
        }
        ++launches;
        g_pack_launches.fetch_add(1, std::memory_order_relaxed);
        g_pack_members.fetch_add((uint64_t)n, std::memory_order_relaxed);
        g_pack.held -= n;
        done += (size_t)n;
    }
    list.erase(list.begin(), list.begin() + (long)done);   // what went out leaves the list on every path
    return failed ? -1 : launches;
}

bool pack_hold(const paella_conv_plan* const* plans, const ConvArgs* args, int n, void* stream, const paella::PoolArgs* pool = nullptr,
               unsigned pool_grid = 0) {
    if (paella::g_pack_recording) {
        if (n != 1 || pool || stream != g_pack.rec_queue) return false;  // the caller's launch then ends the recording
        SeqRecord r;
        r.kind = kMemberConv;
        r.kw = plans[0]->kw;
        r.k_order = plans[0]->k_order ? 1 : 0;
        r.dyn_lds = plans[0]->dims.lds_bytes;
        r.units = plans[0]->dims.grid;
        r.m.conv = args[0];
        g_pack.rec.recs.push_back(r);
        return true;
    }
    if (!g_pack.enabled || paella::timing_events().start != nullptr) return false;
    paella::DirectQueue* q = paella::direct_queue_lookup(stream);
    if (!q || paella::direct_queue_ordered(q)) return false;
    PackList& list = g_pack.lists[kw_index(plans[0]->kw)][plans[0]->k_order ? 1 : 0];
    list.items.emplace_back();
    PackItem& it = list.items.back();
    it.n = n;
    for (int i = 0; i < n; ++i) {
        it.args[i] = args[i];
        it.grids[i] = plans[i]->dims.grid;
        it.grid += plans[i]->dims.grid;
        it.dyn_lds = std::max(it.dyn_lds, plans[i]->dims.lds_bytes);
    }
    if (pool) {
        it.has_pool = true;
        it.pool = *pool;
        it.pool_grid = pool_grid;
        it.grid += pool_grid;
        it.pool.hook_blocks = it.grid;
    }
    for (int i = 0; i < n; ++i) it.args[i].hook_blocks = it.grid;
    list.members += it.members();
    if (g_pack.held++ == 0) g_pack.first_held_ns = now_ns();
    return true;
}

// Sends the held items of one list, oldest first, as few launches as kPackMax problems per launch allow; with
// only_full, stops before a launch that would go out with room to spare.
int pack_send(PackList& list, int kw, int k_order, bool only_full) {
    int launches = 0;
    size_t done = 0;
    bool failed = false;
    while (done < list.items.size()) {
        if (only_full && list.members < kPackMax) break;
        ConvGroupArgs g;
        int n = 0;
        unsigned grid = 0, dyn_lds = 0;
        size_t i = done;
        int total = 0;
        for (; i < list.items.size() && total + list.items[i].members() <= kPackMax; ++i) total += list.items[i].members();
        g.kinds = 0;
        for (size_t k = done; k < i; ++k) {  // the convs of every item first ...
            const PackItem& it = list.items[k];
            for (int c = 0; c < it.n; ++c) {
                grid = align_start(grid);
                g.m[n].conv = it.args[c];
                g.start[n] = grid;
                grid += it.grids[c];
                ++n;
            }
            dyn_lds = std::max(dyn_lds, it.dyn_lds);
        }
        for (size_t k = done; k < i; ++k) {  // ... then their pooling operators
            const PackItem& it = list.items[k];
            if (!it.has_pool) continue;
            g.m[n].pool = it.pool;
            g.start[n] = grid;
            g.kinds |= kMemberPool << (2 * n);
            grid += it.pool_grid;
            ++n;
        }
        void* target = nullptr;
        int rc = paella_direct_queue_shared(&target) != 0 ? -1 : 0;
        if (rc != 0) {
            failed = true;
            break;
        }
        if (n == 1) {  // nothing to share the launch with: the plain kernel, whose argument block is a quarter of the group's
            ConvKernel kern = pick_kernel(1, 1, kw, k_order);
            g.m[0].conv.hook_blocks = grid;
            rc = allow_lds(reinterpret_cast<const void*>(kern), dyn_lds);
            if (rc == 0) {
                paella::launch(kern, dim3(grid), dim3(64u * (unsigned)kw), dyn_lds, reinterpret_cast<hipStream_t>(target), g.m[0].conv);
                rc = (int)hipGetLastError();
            }
        } else {
            rc = launch_group_args(g, n, kw, k_order, grid, dyn_lds, target);
        }
        if (rc != 0) {
            failed = true;
            break;
        }
        ++launches;
        g_pack_launches.fetch_add(1, std::memory_order_relaxed);
        g_pack_members.fetch_add((uint64_t)n, std::memory_order_relaxed);
        for (size_t k = done; k < i; ++k) list.members -= list.items[k].members();
        g_pack.held -= (int)(i - done);
        done = i;
    }
    // what went out leaves the list on every path: a failed launch must not send its predecessors again on the next turn
    list.items.erase(list.items.begin(), list.items.begin() + (long)done);
    return failed ? -1 : launches;
}

unsigned units_to_grid(const SeqRecord& r) {
    if (r.kind == kMemberPool) return (r.units + 255u) / 256u;  // one element per thread
    if (r.kind == kMemberDense) return (r.units + 3u) / 4u;     // one row per wave
    return r.units;
}

// The k-th launches of seqs[first .. first + n) as one grid on `queue`; a member with a notifier reports its own workgroups.
int seq_launch_position(const std::vector<Sequence>& seqs, size_t first, int n, size_t k, void* queue) {
    const SeqRecord& head = seqs[first].recs[k];
    ConvGroupArgs g;
    g.kinds = 0;
    unsigned grid = 0, dyn_lds = 0;
    for (int i = 0; i < n; ++i) {
        const SeqRecord& r = seqs[first + (size_t)i].recs[k];
        const unsigned wgs = units_to_grid(r);
        if (r.kind == kMemberConv) grid = align_start(grid);
        g.m[i] = r.m;
        if (r.kind == kMemberConv) g.m[i].conv.hook_blocks = wgs;
        else if (r.kind == kMemberPool) g.m[i].pool.hook_blocks = wgs;
        else g.m[i].dense.hook_blocks = wgs;
        g.kinds |= r.kind << (2 * i);
        g.start[i] = grid;
        grid += wgs;
        dyn_lds = std::max(dyn_lds, r.dyn_lds);
    }
    g_pack_launches.fetch_add(1, std::memory_order_relaxed);
    g_pack_members.fetch_add((uint64_t)n, std::memory_order_relaxed);
    if (n == 1 && head.kind == kMemberConv) {
        ConvKernel kern = pick_kernel(1, 1, head.kw, head.k_order);
        g.m[0].conv.hook_blocks = grid;
        if (int rc = allow_lds(reinterpret_cast<const void*>(kern), dyn_lds)) return rc;
        paella::launch(kern, dim3(grid), dim3(64u * (unsigned)head.kw), dyn_lds, reinterpret_cast<hipStream_t>(queue), g.m[0].conv);
        return (int)hipGetLastError();
    }
    return launch_group_args(g, n, head.kw, head.k_order, grid, dyn_lds, queue);
}

// Sends seqs[first .. first + n) position by position on one queue of the shared set, with the barrier bit set.
int seq_send_batch(const std::vector<Sequence>& seqs, size_t first, int n, void* queue) {
    void* target = queue;
    if (!target && paella_direct_queue_shared(&target) != 0) return -1;
    paella::DirectQueue* q = paella::direct_queue_lookup(target);
    if (!q) return -1;
    const bool was_ordered = paella::direct_queue_ordered(q);
    paella_direct_queue_set_ordered(target, 1);
    int launches = 0;
    bool failed = false;
    for (size_t k = 0; k < seqs[first].recs.size() && !failed; ++k) {
        if (seq_launch_position(seqs, first, n, k, target) != 0) failed = true;
        else ++launches;
    }
    if (!was_ordered) paella_direct_queue_set_ordered(target, 0);   // on every path: the queue is shared
    return failed ? -1 : launches;
}

int seq_send(SeqList& list, bool only_full) {
    int launches = 0;
    size_t done = 0;
    bool failed = false;
    while (done < list.seqs.size()) {
        const size_t left = list.seqs.size() - done;
        if (only_full && left < (size_t)kPackMax) break;
        const int n = (int)std::min<size_t>(left, (size_t)kPackMax);
        const int r = seq_send_batch(list.seqs, done, n, nullptr);
        // a batch that failed part of the way is gone too: its first launches are on the queue and cannot be sent again
        done += (size_t)n;
        g_pack.held -= n;
        if (r < 0) {
            failed = true;
            break;
        }
        launches += r;
    }
    list.seqs.erase(list.seqs.begin(), list.seqs.begin() + (long)done);
    return failed ? -1 : launches;
}

bool same_signature(const Sequence& a, const Sequence& b) {
    if (a.recs.size() != b.recs.size()) return false;
    for (size_t k = 0; k < a.recs.size(); ++k)
        if (a.recs[k].kind != b.recs[k].kind || a.recs[k].kw != b.recs[k].kw || a.recs[k].k_order != b.recs[k].k_order) return false;
    return true;
}

int pre_send_all(bool only_full);  // below, with the kernels it launches
int dw_send_all(bool only_full);

int pack_send_all(bool only_full) {
    int launches = 0;
    {
        const int r = pre_send_all(only_full);
        if (r < 0) return PAELLA_ENOSUP;
        launches += r;
    }
    {
        const int r = dw_send_all(only_full);
        if (r < 0) return PAELLA_ENOSUP;
        launches += r;
    }
    for (SeqList& list : g_pack.seq_lists) {
        if (list.seqs.empty()) continue;
        const int r = seq_send(list, only_full);
        if (r < 0) return PAELLA_ENOSUP;
        launches += r;
    }
    for (int w = 0; w < 4; ++w)
        for (int o = 0; o < 2; ++o) {
            PackList& list = g_pack.lists[w][o];
            if (list.items.empty()) continue;
            const int r = pack_send(list, 1 << w, o, only_full);
            if (r < 0) return PAELLA_ENOSUP;
            launches += r;
        }
    if (g_pack.held > 0 && !only_full) g_pack.first_held_ns = now_ns();
    return launches;
}

}  // namespace

namespace paella {

thread_local bool g_pack_recording = false;

bool pack_record_pool(const PoolArgs& a, void* stream) {
    if (!g_pack_recording || stream != g_pack.rec_queue) return false;
    SeqRecord r;
    r.kind = kMemberPool;
    r.units = (unsigned)((size_t)a.C * a.P * a.Q);
    r.m.pool = a;
    g_pack.rec.recs.push_back(r);
    return true;
}

bool pack_record_dense(const DenseArgs& a, void* stream) {
    if (!g_pack_recording || stream != g_pack.rec_queue) return false;
    SeqRecord r;
    r.kind = kMemberDense;
    r.units = (unsigned)a.O;
    r.m.dense = a;
    g_pack.rec.recs.push_back(r);
    return true;
}

void pack_sequence_break_slow() {
    g_pack_recording = false;  // first: the launches below go through the same launch path
    if (!g_pack.rec.recs.empty()) {
        std::vector<Sequence> one(1);
        one[0].recs.swap(g_pack.rec.recs);
        if (seq_send_batch(one, 0, 1, g_pack.rec_queue) < 0) {
            std::fprintf(stderr, "[paella] launch packing: a recorded sequence could not be sent\n");
            std::abort();
        }
    }
}

}  // namespace paella

extern "C" int paella_pack_sequence_begin(const void* key, void* queue) {
    if (paella::g_pack_recording) return PAELLA_EINVAL;
    paella::DirectQueue* q = paella::direct_queue_lookup(queue);
    if (!g_pack.enabled || !q || !paella::direct_queue_ordered(q) || paella::timing_events().start != nullptr) return PAELLA_ENOSUP;
    g_pack.rec_key = key;
    g_pack.rec_queue = queue;
    g_pack.rec.recs.clear();
    paella::g_pack_recording = true;
    return 0;
}

extern "C" int paella_pack_sequence_end(void) {
    if (!paella::g_pack_recording) return 0;  // never begun, or ended by a launch the recorder does not take: all sent already
    paella::g_pack_recording = false;
    if (g_pack.rec.recs.empty()) return 0;
    SeqList* list = nullptr;
    for (SeqList& l : g_pack.seq_lists)
        if (l.key == g_pack.rec_key) list = &l;
    if (!list) {
        g_pack.seq_lists.emplace_back();
        list = &g_pack.seq_lists.back();
        list->key = g_pack.rec_key;
    }
    if (!list->seqs.empty() && !same_signature(list->seqs.front(), g_pack.rec)) {
        if (seq_send(*list, false) < 0) return PAELLA_ENOSUP;
    }
    list->seqs.emplace_back();
    list->seqs.back().recs.swap(g_pack.rec.recs);
    if (g_pack.held++ == 0) g_pack.first_held_ns = now_ns();
    return 0;
}

extern "C" int paella_pack_enable(int on) {
    if (!on && g_pack.held > 0) {
        if (int rc = pack_send_all(false); rc < 0) return rc;
    }
    g_pack.enabled = on != 0;
    return 0;
}

extern "C" int paella_pack_flush(void) { return g_pack.held > 0 ? pack_send_all(false) : 0; }

extern "C" int paella_pack_poll(void) {
    if (g_pack.held == 0) return 0;
    if (paella::direct_shared_min_waiting() == 0 || now_ns() - g_pack.first_held_ns >= kPackHoldNs) return pack_send_all(false);
    return pack_send_all(true);
}

extern "C" void paella_pack_poll_hook(void) {
    // Held launches that cannot be sent leave their requests without completion messages for good: nothing the serving loop
    // could do about it but stop, loudly.
    if (paella_pack_poll() < 0) {
        std::fprintf(stderr, "[paella] launch packing: held launches could not be sent\n");
        std::abort();
    }
}

extern "C" int paella_pack_stats(uint64_t* launches, uint64_t* members) {
    if (launches) *launches = g_pack_launches.load(std::memory_order_relaxed);
    if (members) *members = g_pack_members.load(std::memory_order_relaxed);
    return g_pack.held;
}

extern "C" int paella_conv2d_launch_group(const paella_conv_operands* members, int n, void* stream, uint32_t job_id, void* notifier) {
    if (!members || n < 2 || n > kMaxGroup) return PAELLA_EINVAL;
    const paella_conv_plan* plans[kMaxGroup];
    for (int i = 0; i < n; ++i) plans[i] = members[i].plan;
    paella_launch_dims dims;
    if (int rc = paella_conv2d_group_dims(plans, n, &dims)) return rc;
    for (int i = 0; i < n; ++i)  // two split reductions must not share their counters and partial tiles
        for (int j = i + 1; j < n; ++j)
            if (plans[i]->splits > 1 && plans[j]->splits > 1 && members[i].workspace == members[j].workspace) return PAELLA_EINVAL;
    auto* nf = reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier);
    ConvGroupArgs g;
    ConvArgs args[kMaxGroup];
    unsigned next = 0, dyn_lds = 0;  // dims.lds_bytes is the scheduler's figure and includes the kernel's static LDS
    for (int i = 0; i < n; ++i) {
        const paella_conv_operands& m = members[i];
        if (int rc = fill_args(m.plan, m.x, m.blob_dev, m.bias, m.residual, m.slope, m.y, m.workspace, job_id, nf, args[i])) return rc;
        dyn_lds = std::max(dyn_lds, m.plan->dims.lds_bytes);
    }
    if (pack_hold(plans, args, n, stream)) return 0;
    for (int i = 0; i < n; ++i) {
        next = align_start(next);
        g.m[i].conv = args[i];
        g.m[i].conv.hook_blocks = dims.grid;  // the launch is longer than the workgroups that report: ids skipped by align_start
        g.start[i] = next;
        next += plans[i]->dims.grid;
    }
    g.kinds = 0;
    return launch_group_args(g, n, plans[0]->kw, plans[0]->k_order, next, dyn_lds, stream);
}

extern "C" int paella_conv2d_group_pool_dims(const paella_conv_plan* const* plans, int n, const paella_pool_desc* pool, paella_launch_dims* dims) {
    if (!plans || n < 1 || n > kMaxGroupWithPool || !pool) return PAELLA_EINVAL;
    for (int i = 0; i < n; ++i) {
        if (!plans[i]) return PAELLA_EINVAL;
        const paella_conv_plan& p = *plans[i];
        if (p.kind != 0 || p.mi != 1 || p.ni != 1 || p.kw != plans[0]->kw || p.k_order != 1) return PAELLA_ENOSUP;
    }
    paella::PoolArgs pa;
    if (!paella::pool_fill_args(pool, nullptr, nullptr, 0, nullptr, &pa)) return PAELLA_EINVAL;
    if (dims) {
        dims->grid = 0;
        dims->lds_bytes = 0;
        for (int i = 0; i < n; ++i) {
            dims->grid += plans[i]->dims.grid;
            if (plans[i]->dims.lds_bytes > dims->lds_bytes) dims->lds_bytes = plans[i]->dims.lds_bytes;
        }
        dims->block = plans[0]->dims.block;
        dims->grid += (unsigned)(((size_t)pa.C * pa.P * pa.Q + dims->block - 1) / dims->block);
        dims->vgprs = plans[0]->dims.vgprs;
        add_kernel_resources(reinterpret_cast<const void*>(pick_group_kernel(plans[0]->kw, 1)), dims);
    }
    return 0;
}

extern "C" int paella_conv2d_launch_group_pool(const paella_conv_operands* members, int n, const paella_pool_desc* pool, const float* pool_x,
                                               float* pool_y, void* stream, uint32_t job_id, void* notifier) {
    if (!members || n < 1 || n > kMaxGroupWithPool || !pool || !pool_x || !pool_y) return PAELLA_EINVAL;
    const paella_conv_plan* plans[kMaxGroupWithPool];
    for (int i = 0; i < n; ++i) plans[i] = members[i].plan;
    paella_launch_dims dims;
    if (int rc = paella_conv2d_group_pool_dims(plans, n, pool, &dims)) return rc;
    for (int i = 0; i < n; ++i)
        for (int j = i + 1; j < n; ++j)
            if (plans[i]->splits > 1 && plans[j]->splits > 1 && members[i].workspace == members[j].workspace) return PAELLA_EINVAL;
    auto* nf = reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier);
    ConvGroupArgs g;
    ConvArgs args[kMaxGroupWithPool];
    unsigned next = 0, dyn_lds = 0;  // dims.lds_bytes is the scheduler's figure and includes the kernel's static LDS
    for (int i = 0; i < n; ++i) {
        const paella_conv_operands& m = members[i];
        if (int rc = fill_args(m.plan, m.x, m.blob_dev, m.bias, m.residual, m.slope, m.y, m.workspace, job_id, nf, args[i])) return rc;
        next += m.plan->dims.grid;
        dyn_lds = std::max(dyn_lds, m.plan->dims.lds_bytes);
    }
    paella::PoolArgs pa;
    if (!paella::pool_fill_args(pool, pool_x, pool_y, job_id, notifier, &pa)) return PAELLA_EINVAL;
    const unsigned pool_grid = dims.grid - next;
    if (pack_hold(plans, args, n, stream, &pa, pool_grid)) return 0;
    next = 0;
    for (int i = 0; i < n; ++i) {
        next = align_start(next);
        g.m[i].conv = args[i];
        g.m[i].conv.hook_blocks = dims.grid;  // the launch is longer than the workgroups that report: ids skipped by align_start
        g.start[i] = next;
        next += plans[i]->dims.grid;
    }
    pa.hook_blocks = dims.grid;
    g.m[n].pool = pa;
    g.start[n] = next;
    g.kinds = kMemberPool << (2 * n);
    return launch_group_args(g, n + 1, plans[0]->kw, 1, next + pool_grid, dyn_lds, stream);
}

extern "C" int paella_conv2d_pair_dims(const paella_conv_plan* first, const paella_conv_plan* second, paella_launch_dims* dims) {
    const paella_conv_plan* plans[2] = {first, second};
    return paella_conv2d_group_dims(plans, 2, dims);
}

extern "C" int paella_conv2d_launch_pair(const paella_conv_operands* first, const paella_conv_operands* second, void* stream, uint32_t job_id,
                                         void* notifier) {
    if (!first || !second) return PAELLA_EINVAL;
    const paella_conv_operands members[2] = {*first, *second};
    return paella_conv2d_launch_group(members, 2, stream, job_id, notifier);
}

extern "C" int paella_conv2d_launch(const paella_conv_plan* plan, const float* x, const void* blob_dev, const float* bias,
                                    const float* residual, const float* slope, float* y, void* workspace, void* stream,
                                    uint32_t job_id, void* notifier) {
    if (!plan || !x || !blob_dev || !y) return PAELLA_EINVAL;
    const paella_conv_desc& d = plan->d;
    if (d.act == PAELLA_ACT_PRELU && !slope) return PAELLA_EINVAL;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    auto* nf = reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier);
    const int PQ = plan->P * plan->Q;
    if (plan->kind == 0) {
        ConvKernel kern = pick_kernel(plan->mi, plan->ni, plan->kw, plan->k_order, plan->depth);
        if (!kern) return PAELLA_EINVAL;
        ConvArgs a;
        if (int rc = fill_args(plan, x, blob_dev, bias, residual, slope, y, workspace, job_id, nf, a)) return rc;
        if (plan->mi == 1 && plan->ni == 1 && !plan->depth && pack_hold(&plan, &a, 1, stream)) return 0;
        if (int rc = allow_lds(reinterpret_cast<const void*>(kern), plan->dims.lds_bytes)) return rc;
        paella::launch(kern, dim3(plan->dims.grid), dim3(plan->dims.block), plan->dims.lds_bytes, st, a);
        return (int)hipGetLastError();
    }
    DwArgs a;
    a.x = x; a.w = reinterpret_cast<const float*>(blob_dev); a.bias = bias; a.residual = residual; a.slope = slope; a.y = y;
    a.C = d.C; a.H = d.H; a.W = d.W; a.P = plan->P; a.Q = plan->Q; a.R = d.R; a.S = d.S;
    a.sh = d.stride_h; a.sw = d.stride_w; a.ph = d.pad_h; a.pw = d.pad_w; a.dh = d.dil_h; a.dw = d.dil_w;
    a.act = d.act; a.lo = d.act_lo; a.hi = d.act_hi;
    a.job_id = job_id;
    a.notifier = nf;
    {
        // The batched 3 x 3 form: divisions by multiply-high are exact while dividend x divisor < 2^32 (elements by Q, rows by P),
        // offsets are 32-bit byte offsets, coordinates go through 24-bit multiplies.
        const uint64_t elements = (uint64_t)d.C * plan->P * plan->Q, rows = (uint64_t)d.C * plan->P;
        const uint64_t x_bytes = (uint64_t)d.C * d.H * d.W * 4, pad = ((uint64_t)d.pad_h * d.W + d.pad_w) * 4;
        a.fast = d.R == 3 && d.S == 3 && elements * (uint64_t)plan->Q < ((uint64_t)1 << 32) && rows * (uint64_t)plan->P < ((uint64_t)1 << 32) &&
                 x_bytes + pad + (uint64_t)(2 * d.dil_h * d.W + 2 * d.dil_w) * 4 < ((uint64_t)1 << 31) && elements * 4 < ((uint64_t)1 << 31) &&
                 elements < (1u << 23) && (uint64_t)d.C * d.H < (1u << 23) && d.W < (1 << 23) && plan->Q < (1 << 23) ? 1 : 0;
        a.div_q = fast_div((unsigned)plan->Q);
        a.div_p = fast_div((unsigned)plan->P);
        a.x_bytes = (unsigned)std::min<uint64_t>(x_bytes, 0xFFFFFFFFu);
        a.out_bytes = (unsigned)std::min<uint64_t>(elements * 4, 0xFFFFFFFFu);
    }
    if (pack_hold_dw(a, plan->dims.grid, stream)) return 0;
    paella::launch(dwconv_kernel, dim3(plan->dims.grid), dim3(256), 0, st, a);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Allocation-free variant: the split-reduction workspace is a fixed array of the device image.  The array's name is a
// host-side handle, not a device address: each GPU holds its own copy, whose address is looked up once per device.

static __device__ __align__(256) unsigned char scratch[PAELLA_CONV_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned* p, unsigned n) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// Device address of this GPU's copy of `scratch` (looked up on the first call per device, with that device current).
int static_workspace(void** out) {
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev)) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return PAELLA_ENOSUP;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return (int)e;
            if (!p) return (int)hipErrorInvalidSymbol;
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return 0;
}

}  // namespace

extern "C" int paella_conv2d_static_init(void) {
    void* ws = nullptr;
    return static_workspace(&ws);
}

extern "C" int paella_conv2d_static_workspace(void** ptr) {
    if (!ptr) return PAELLA_EINVAL;
    return static_workspace(ptr);
}

extern "C" int paella_conv2d_launch_static(const paella_conv_plan* plan, const float* x, const void* blob_dev, const float* bias,
                                           const float* residual, const float* slope, float* y, void* stream, uint32_t job_id,
                                           void* notifier) {
    if (!plan || !x || !blob_dev || !y) return PAELLA_EINVAL;
    if (plan->d.act == PAELLA_ACT_PRELU && !slope) return PAELLA_EINVAL;
    if (plan->workspace_bytes > PAELLA_CONV_STATIC_WORKSPACE_BYTES) return PAELLA_ETOOBIG;
    if (paella::direct_queue_lookup(stream)) return PAELLA_ENOSUP;  // the counter fill below needs stream order
    void* ws = nullptr;
    if (plan->workspace_bytes) {
        if (int rc = static_workspace(&ws)) return rc;
        // Everything the launch itself would refuse is refused here, before the fill kernel goes out.
        if (plan->kind != 0 || plan->splits < 1 || !pick_kernel(plan->mi, plan->ni, plan->kw, plan->k_order, plan->depth)) return PAELLA_EINVAL;
        ConvArgs probe;
        if (int rc = fill_args(plan, x, blob_dev, bias, residual, slope, y, ws, job_id,
                               reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier), probe))
            return rc;
        // One arrival counter per output tile, at the head of the workspace.
        const unsigned tiles = plan->dims.grid / (unsigned)plan->splits;
        hipLaunchKernelGGL(zero_words_kernel, dim3((tiles + 255u) / 256u), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                           reinterpret_cast<unsigned*>(ws), tiles);
        if (hipError_t e = hipGetLastError()) return (int)e;
    }
    return paella_conv2d_launch(plan, x, blob_dev, bias, residual, slope, y, ws, stream, job_id, notifier);
}

typedef void (*ConvPreKernel)(ConvPreArgs);

static ConvPreKernel pick_pre_kernel(int kw) {
    switch (kw) {
        case 1: return conv_mfma_pre_kernel<1>;
        case 2: return conv_mfma_pre_kernel<2>;
        case 4: return conv_mfma_pre_kernel<4>;
        case 8: return conv_mfma_pre_kernel<8>;
        default: return nullptr;
    }
}

namespace {

typedef void (*ConvPreGroupKernel)(ConvPreGroupArgs);

ConvPreGroupKernel pick_pre_group_kernel(int kw) {
    switch (kw) {
        case 1: return conv_mfma_pre_group_kernel<1>;
        case 2: return conv_mfma_pre_group_kernel<2>;
        case 4: return conv_mfma_pre_group_kernel<4>;
        case 8: return conv_mfma_pre_group_kernel<8>;
        default: return nullptr;
    }
}

// Dynamic LDS of a launch with a fused input transform: the plan's (the partial tiles of the cross-wave sum) and behind it the
// table of scales and shifts -- 64 bytes of zeros and 8 bytes per input channel.
unsigned pre_lds_bytes(const paella_conv_plan* plan) { return plan->dims.lds_bytes + 64u + 8u * (unsigned)((plan->d.C + 7) / 8 * 8); }

// Launch packing of convs with a fused input transform: held like the plain ones (pack_hold), in lists of their own
// because they run in a kernel of their own.
bool pack_hold_pre(const paella_conv_plan* plan, const ConvPreArgs& a, void* stream) {
    if (paella::g_pack_recording || !g_pack.enabled || paella::timing_events().start != nullptr) return false;
    paella::DirectQueue* q = paella::direct_queue_lookup(stream);
    if (!q || paella::direct_queue_ordered(q)) return false;
    PackState::PreItem it;
    it.a = a;
    it.grid = plan->dims.grid;
    it.dyn_lds = pre_lds_bytes(plan);
    it.a.conv.hook_blocks = it.grid;
    g_pack.pre_lists[kw_index(plan->kw)].push_back(it);
    if (g_pack.held++ == 0) g_pack.first_held_ns = now_ns();
    return true;
}

int pre_send_all(bool only_full) {
    int launches = 0;
    for (int w = 0; w < 4; ++w) {
        std::vector<PackState::PreItem>& list = g_pack.pre_lists[w];
        size_t done = 0;
        const int kw = 1 << w;
        while (done < list.size()) {
            const size_t left = list.size() - done;
            if (only_full && left < (size_t)kPackMax) break;
            const int n = (int)std::min<size_t>(left, (size_t)kPackMax);
            void* target = nullptr;
            unsigned grid = 0, dyn_lds = 0;
            int rc = paella_direct_queue_shared(&target) != 0 ? -1 : 0;
            if (rc != 0) {
            } else if (n == 1) {
                ConvPreKernel kern = pick_pre_kernel(kw);
                ConvPreArgs a = list[done].a;
                a.conv.hook_blocks = list[done].grid;
                rc = allow_lds(reinterpret_cast<const void*>(kern), list[done].dyn_lds);
                if (rc == 0) {
                    paella::launch(kern, dim3(list[done].grid), dim3(64u * (unsigned)kw), list[done].dyn_lds, reinterpret_cast<hipStream_t>(target), a);
                    rc = (int)hipGetLastError();
                }
            } else {
                ConvPreGroupArgs g;
                for (int i = 0; i < n; ++i) {
                    grid = align_start(grid);
                    g.m[i] = list[done + (size_t)i].a;
                    g.start[i] = grid;
                    grid += list[done + (size_t)i].grid;
                    dyn_lds = std::max(dyn_lds, list[done + (size_t)i].dyn_lds);
                }
                for (int i = n; i < kPackMax; ++i) g.start[i] = 0xFFFFFFFFu;
                ConvPreGroupKernel kern = pick_pre_group_kernel(kw);
                rc = allow_lds(reinterpret_cast<const void*>(kern), dyn_lds);
                if (rc == 0) {
                    paella::launch_used(kern, dim3(grid), dim3(64u * (unsigned)kw), dyn_lds, reinterpret_cast<hipStream_t>(target),
                                        offsetof(ConvPreGroupArgs, m) + (size_t)n * sizeof(ConvPreArgs), g);
                    rc = (int)hipGetLastError();
                }
            }
            if (rc != 0) {  // what went out before leaves the list all the same
                list.erase(list.begin(), list.begin() + (long)done);
                return -1;
            }
            ++launches;
            g_pack_launches.fetch_add(1, std::memory_order_relaxed);
            g_pack_members.fetch_add((uint64_t)n, std::memory_order_relaxed);
            g_pack.held -= n;
            done += (size_t)n;
        }
        list.erase(list.begin(), list.begin() + (long)done);
    }
    return launches;
}

}  // namespace

extern "C" int paella_conv2d_plan_takes_input_transform(const paella_conv_plan* plan) {
    return plan && plan->kind == 0 && plan->mi == 1 && plan->ni == 1 && plan->k_order == 1 ? 1 : 0;
}

extern "C" int paella_conv2d_transformed_dims(const paella_conv_plan* plan, paella_launch_dims* dims) {
    if (!plan || !dims) return PAELLA_EINVAL;
    if (!paella_conv2d_plan_takes_input_transform(plan)) return PAELLA_ENOSUP;
    *dims = plan->dims;
    dims->lds_bytes = pre_lds_bytes(plan);
    add_kernel_resources(reinterpret_cast<const void*>(pick_pre_kernel(plan->kw)), dims);
    return 0;
}

extern "C" int paella_conv2d_dims(const paella_conv_plan* plan, paella_launch_dims* dims) {
    if (!plan || !dims) return PAELLA_EINVAL;
    *dims = plan->dims;
    add_kernel_resources(plan->kind == 1 ? reinterpret_cast<const void*>(dwconv_kernel)
                                         : reinterpret_cast<const void*>(pick_kernel(plan->mi, plan->ni, plan->kw, plan->k_order, plan->depth)), dims);
    return 0;
}

extern "C" int paella_conv2d_launch_transformed(const paella_conv_plan* plan, const float* x, const float* in_scale, const float* in_shift,
                                                int in_act, const void* blob_dev, const float* bias, const float* residual,
                                                const float* slope, float* y, void* workspace, void* stream, uint32_t job_id,
                                                void* notifier) {
    if (!plan || !x || !in_scale || !in_shift || !blob_dev || !y) return PAELLA_EINVAL;
    if (in_act != PAELLA_ACT_NONE && in_act != PAELLA_ACT_RELU) return PAELLA_EINVAL;
    if (!paella_conv2d_plan_takes_input_transform(plan)) return PAELLA_ENOSUP;
    ConvPreKernel kern = pick_pre_kernel(plan->kw);
    if (!kern) return PAELLA_EINVAL;
    ConvPreArgs a;
    if (int rc = fill_args(plan, x, blob_dev, bias, residual, slope, y, workspace, job_id,
                           reinterpret_cast<llis::job::FinishedBlockNotifier*>(notifier), a.conv))
        return rc;
    a.pre.scale = in_scale;
    a.pre.shift = in_shift;
    a.pre.lo = in_act == PAELLA_ACT_RELU ? 0.f : -__builtin_inff();
    if (pack_hold_pre(plan, a, stream)) return 0;
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), pre_lds_bytes(plan))) return rc;
    paella::launch(kern, dim3(plan->dims.grid), dim3(plan->dims.block), pre_lds_bytes(plan), reinterpret_cast<hipStream_t>(stream), a);
    return (int)hipGetLastError();
}

extern "C" int paella_conv_kernel_occupancy(int kind, int form, int mi, int ni, int kw, int k_order, unsigned lds_bytes, int* blocks_per_cu,
                                            unsigned* vgprs, unsigned* static_lds) {
    if (!blocks_per_cu) return PAELLA_EINVAL;
    const void* fn = nullptr;
    unsigned block = 64u * (unsigned)kw;
    if (kind == 1) {
        fn = reinterpret_cast<const void*>(dwconv_kernel);
        block = 256;
    } else if (form == 0) {
        fn = reinterpret_cast<const void*>(pick_kernel(mi, ni, kw, k_order));
    } else if (mi == 1 && ni == 1) {
        if (form == 1 && k_order == 1) fn = reinterpret_cast<const void*>(pick_pre_kernel(kw));
        else if (form == 2) fn = reinterpret_cast<const void*>(pick_group_kernel(kw, k_order));
        else if (form == 3 && k_order == 1) fn = reinterpret_cast<const void*>(pick_group_kernel(kw, 1));
    }
    if (!fn) return PAELLA_EINVAL;
    if (int rc = allow_lds(fn, lds_bytes)) return rc;
    if (vgprs || static_lds) {
        hipFuncAttributes attr;
        if (hipError_t e = hipFuncGetAttributes(&attr, fn)) return (int)e;
        if (vgprs) *vgprs = (unsigned)attr.numRegs;
        if (static_lds) *static_lds = (unsigned)attr.sharedSizeBytes;
    }
    return (int)hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, fn, (int)block, lds_bytes);
}

extern "C" int paella_conv_kernel_vgprs(int kind, int mi, int ni, int kw, unsigned* vgprs) {
    // the tap-major twin of a variant uses no more registers than the table variant reported here
    const void* fn = kind == 1 ? reinterpret_cast<const void*>(dwconv_kernel) : reinterpret_cast<const void*>(pick_kernel(mi, ni, kw));
    if (!fn || !vgprs) return PAELLA_EINVAL;
    hipFuncAttributes attr;
    hipError_t e = hipFuncGetAttributes(&attr, fn);
    if (e != hipSuccess) return (int)e;
    *vgprs = (unsigned)attr.numRegs;
    return 0;
}
