/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the fp32 NCHW operator set of the serving hot path.
 *
 * Nothing in the product (paella_amd/, include/) may link, import or execute this file; it is the
 * checker used by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py.
 *
 * What it restates: the arithmetic that the reference obtains from its TVM-generated kernels when a job
 * adapter calls run_() (reference jobs/tvm_mnist/tvm_mnist.cpp:41 and the ten sibling adapters).  That
 * generator is the third-party dependency eniac/tvm-llis, tag v0.10.0-llis
 * (reference sosp23_artifact/setup/install_llis_tvm.sh:45-48); it is not vendored, so the operators are
 * restated from their published ONNX/Relay definitions:
 *   conv2d (groups, stride, pad, dilation)    ONNX Conv
 *   dense                                     ONNX Gemm (transB=1)
 *   max/avg pool, global avg pool             ONNX MaxPool / AveragePool / GlobalAveragePool
 *   add, per-channel scale-shift, activations ONNX Add / BatchNormalization(inference) / Relu / Clip / PRelu
 *   softmax, LRN                              ONNX Softmax / LRN
 *
 * Pinning: the reference holds no numeric golden vectors for this path.  Every function here is pinned in
 * tests/test_oracle_ops.py against torch.nn.functional on the CPU (third-party, independent) and against
 * closed forms (identity kernel, zero weight => bias, linearity, output-size formula).
 *
 * All accumulation is in double and rounded once to float, so the oracle is the "true" fp32 answer and the
 * GPU path is compared to it with max-abs 1e-4 / rel 1e-3.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <float.h>

enum { ORC_ACT_NONE = 0, ORC_ACT_RELU = 1, ORC_ACT_RELU6 = 2, ORC_ACT_PRELU = 3, ORC_ACT_CLIP = 4 };

static inline float orc_act(double v, int act, int ch, const float* slope, float lo, float hi) {
    switch (act) {
        case ORC_ACT_RELU:  return (float)(v > 0 ? v : 0);
        case ORC_ACT_RELU6: return (float)(v < 0 ? 0 : (v > 6 ? 6 : v));
        case ORC_ACT_PRELU: return (float)(v > 0 ? v : v * (double)slope[ch]);
        case ORC_ACT_CLIP:  return (float)(v < lo ? lo : (v > hi ? hi : v));
        default:            return (float)v;
    }
}

/* ONNX Conv output extent: floor((in + 2*pad - dil*(k-1) - 1)/stride) + 1 */
int orc_conv_out(int in, int k, int stride, int pad, int dil) {
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

/* ONNX pooling output extent, with optional ceil mode (last window must start inside input+left pad). */
int orc_pool_out(int in, int k, int stride, int pad, int ceil_mode) {
    int num = in + 2 * pad - k;
    int out;
    if (ceil_mode) {
        out = (num + stride - 1) / stride + 1;
        if ((out - 1) * stride >= in + pad) --out;
    } else {
        out = num / stride + 1;
    }
    return out;
}

/*
 * y[n,k,p,q] = act( bias[k] + sum_{c,r,s} x[n, g*Cg+c, p*sh-ph+r*dh, q*sw-pw+s*dw] * w[k,c,r,s] + residual[n,k,p,q] )
 * w layout [K][C/groups][R][S]; residual and bias may be NULL.
 */
void orc_conv2d(const float* x, const float* w, const float* bias, const float* residual, float* y,
                int N, int C, int H, int W, int K, int R, int S,
                int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                int act, const float* slope, float lo, float hi) {
    const int P = orc_conv_out(H, R, sh, ph, dh);
    const int Q = orc_conv_out(W, S, sw, pw, dw);
    const int Cg = C / groups, Kg = K / groups;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int k = 0; k < K; ++k) {
            const int g = k / Kg;
            for (int p = 0; p < P; ++p) {
                for (int q = 0; q < Q; ++q) {
                    double acc = bias ? (double)bias[k] : 0.0;
                    for (int c = 0; c < Cg; ++c) {
                        const float* xc = x + ((size_t)n * C + (size_t)g * Cg + c) * H * W;
                        const float* wc = w + ((size_t)k * Cg + c) * R * S;
                        for (int r = 0; r < R; ++r) {
                            const int h = p * sh - ph + r * dh;
                            if (h < 0 || h >= H) continue;
                            for (int s = 0; s < S; ++s) {
                                const int ww = q * sw - pw + s * dw;
                                if (ww < 0 || ww >= W) continue;
                                acc += (double)xc[(size_t)h * W + ww] * (double)wc[r * S + s];
                            }
                        }
                    }
                    const size_t o = (((size_t)n * K + k) * P + p) * Q + q;
                    if (residual) acc += (double)residual[o];
                    y[o] = orc_act(acc, act, k, slope, lo, hi);
                }
            }
        }
    }
}

/*
 * Throughput-oriented variant of the same definition, used only to TIME the CPU path: float accumulation,
 * inner loop over the output row so the compiler vectorises it.  Results are within fp32 rounding of
 * orc_conv2d (checked in tests/test_oracle_ops.py); it is never used as the parity reference.
 */
void orc_conv2d_fast(const float* x, const float* w, const float* bias, const float* residual, float* y,
                     int N, int C, int H, int W, int K, int R, int S,
                     int sh, int sw, int ph, int pw, int dh, int dw, int groups,
                     int act, const float* slope, float lo, float hi) {
    const int P = orc_conv_out(H, R, sh, ph, dh);
    const int Q = orc_conv_out(W, S, sw, pw, dw);
    const int Cg = C / groups, Kg = K / groups;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int k = 0; k < K; ++k) {
            const int g = k / Kg;
            float* yk = y + ((size_t)n * K + k) * P * Q;
            const float b = bias ? bias[k] : 0.f;
            for (int i = 0; i < P * Q; ++i) yk[i] = b;
            for (int c = 0; c < Cg; ++c) {
                const float* xc = x + ((size_t)n * C + (size_t)g * Cg + c) * H * W;
                const float* wc = w + ((size_t)k * Cg + c) * R * S;
                for (int r = 0; r < R; ++r) {
                    for (int s = 0; s < S; ++s) {
                        const float wv = wc[r * S + s];
                        /* valid q range: 0 <= q*sw - pw + s*dw < W */
                        int q0 = 0, q1 = Q;
                        {
                            int off = s * dw - pw;
                            if (off < 0) q0 = (-off + sw - 1) / sw;
                            int lim = W - off; /* q*sw < lim */
                            int qmax = (lim + sw - 1) / sw;
                            if (qmax < q1) q1 = qmax;
                        }
                        for (int p = 0; p < P; ++p) {
                            const int h = p * sh - ph + r * dh;
                            if (h < 0 || h >= H) continue;
                            const float* xr = xc + (size_t)h * W + (s * dw - pw);
                            float* yr = yk + (size_t)p * Q;
                            if (sw == 1) {
                                for (int q = q0; q < q1; ++q) yr[q] += wv * xr[q];
                            } else {
                                for (int q = q0; q < q1; ++q) yr[q] += wv * xr[(size_t)q * sw];
                            }
                        }
                    }
                }
            }
            const float* rk = residual ? residual + ((size_t)n * K + k) * P * Q : NULL;
            for (int i = 0; i < P * Q; ++i) {
                double v = yk[i];
                if (rk) v = (double)(yk[i] + rk[i]);
                yk[i] = orc_act(v, act, k, slope, lo, hi);
            }
        }
    }
}

/* y[n,o] = act(bias[o] + sum_i x[n,i] * w[o,i])   (ONNX Gemm with transB=1) */
void orc_dense(const float* x, const float* w, const float* bias, float* y, int N, int I, int O, int act) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int o = 0; o < O; ++o) {
            double acc = bias ? (double)bias[o] : 0.0;
            const float* xi = x + (size_t)n * I;
            const float* wo = w + (size_t)o * I;
            for (int i = 0; i < I; ++i) acc += (double)xi[i] * (double)wo[i];
            y[(size_t)n * O + o] = orc_act(acc, act, o, NULL, 0, 0);
        }
    }
}

/* Max pool; padding contributes -inf (never selected). */
void orc_maxpool2d(const float* x, float* y, int N, int C, int H, int W,
                   int R, int S, int sh, int sw, int ph, int pw, int ceil_mode) {
    const int P = orc_pool_out(H, R, sh, ph, ceil_mode);
    const int Q = orc_pool_out(W, S, sw, pw, ceil_mode);
#pragma omp parallel for schedule(static)
    for (int nc = 0; nc < N * C; ++nc) {
        const float* xc = x + (size_t)nc * H * W;
        float* yc = y + (size_t)nc * P * Q;
        for (int p = 0; p < P; ++p)
            for (int q = 0; q < Q; ++q) {
                float m = -FLT_MAX;
                for (int r = 0; r < R; ++r) {
                    int h = p * sh - ph + r;
                    if (h < 0 || h >= H) continue;
                    for (int s = 0; s < S; ++s) {
                        int ww = q * sw - pw + s;
                        if (ww < 0 || ww >= W) continue;
                        float v = xc[(size_t)h * W + ww];
                        if (v > m) m = v;
                    }
                }
                yc[(size_t)p * Q + q] = m;
            }
    }
}

/*
 * Average pool.  count_include_pad=1 divides by the window area clipped to input+padding (ONNX/torch
 * semantics with ceil mode), 0 divides by the number of in-bounds taps.
 */
void orc_avgpool2d(const float* x, float* y, int N, int C, int H, int W,
                   int R, int S, int sh, int sw, int ph, int pw, int ceil_mode, int count_include_pad) {
    const int P = orc_pool_out(H, R, sh, ph, ceil_mode);
    const int Q = orc_pool_out(W, S, sw, pw, ceil_mode);
#pragma omp parallel for schedule(static)
    for (int nc = 0; nc < N * C; ++nc) {
        const float* xc = x + (size_t)nc * H * W;
        float* yc = y + (size_t)nc * P * Q;
        for (int p = 0; p < P; ++p)
            for (int q = 0; q < Q; ++q) {
                double acc = 0;
                int valid = 0, padded = 0;
                for (int r = 0; r < R; ++r) {
                    int h = p * sh - ph + r;
                    for (int s = 0; s < S; ++s) {
                        int ww = q * sw - pw + s;
                        if (h < H + ph && ww < W + pw) ++padded;
                        if (h < 0 || h >= H || ww < 0 || ww >= W) continue;
                        acc += (double)xc[(size_t)h * W + ww];
                        ++valid;
                    }
                }
                int div = count_include_pad ? padded : valid;
                yc[(size_t)p * Q + q] = (float)(div ? acc / div : 0.0);
            }
    }
}

void orc_global_avgpool(const float* x, float* y, int N, int C, int HW) {
    for (int nc = 0; nc < N * C; ++nc) {
        double acc = 0;
        for (int i = 0; i < HW; ++i) acc += (double)x[(size_t)nc * HW + i];
        y[nc] = (float)(acc / HW);
    }
}

/* y = act(a + b), elementwise over n values laid out [C][HW] for the per-channel activations. */
void orc_add(const float* a, const float* b, float* y, int C, int HW, int act, const float* slope, float lo, float hi) {
    for (int c = 0; c < C; ++c)
        for (int i = 0; i < HW; ++i) {
            size_t o = (size_t)c * HW + i;
            y[o] = orc_act((double)a[o] + (double)b[o], act, c, slope, lo, hi);
        }
}

/* y[c,i] = act(x[c,i] * scale[c] + shift[c]); scale or shift may be NULL (1 / 0). */
void orc_scale_shift(const float* x, const float* scale, const float* shift, float* y, int C, int HW,
                     int act, const float* slope, float lo, float hi) {
    for (int c = 0; c < C; ++c) {
        double sc = scale ? (double)scale[c] : 1.0, sf = shift ? (double)shift[c] : 0.0;
        for (int i = 0; i < HW; ++i) {
            size_t o = (size_t)c * HW + i;
            y[o] = orc_act((double)x[o] * sc + sf, act, c, slope, lo, hi);
        }
    }
}

/* Softmax over the last axis of a [rows][cols] matrix. */
void orc_softmax(const float* x, float* y, int rows, int cols) {
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * cols;
        float* yr = y + (size_t)r * cols;
        double m = -DBL_MAX;
        for (int i = 0; i < cols; ++i) if (xr[i] > m) m = xr[i];
        double sum = 0;
        for (int i = 0; i < cols; ++i) sum += exp((double)xr[i] - m);
        for (int i = 0; i < cols; ++i) yr[i] = (float)(exp((double)xr[i] - m) / sum);
    }
}

/* ONNX LRN across channels: y = x / (k + alpha/size * sum_{c' in window} x^2)^beta,
 * window = [c - floor((size-1)/2), c + ceil((size-1)/2)] clipped to [0, C). */
void orc_lrn(const float* x, float* y, int C, int HW, int size, float alpha, float beta, float k) {
    const int lo = (size - 1) / 2, hi = size - 1 - lo;
    for (int c = 0; c < C; ++c)
        for (int i = 0; i < HW; ++i) {
            double sq = 0;
            for (int cc = c - lo; cc <= c + hi; ++cc) {
                if (cc < 0 || cc >= C) continue;
                double v = x[(size_t)cc * HW + i];
                sq += v * v;
            }
            double d = pow((double)k + (double)alpha / size * sq, (double)beta);
            y[(size_t)c * HW + i] = (float)((double)x[(size_t)c * HW + i] / d);
        }
}

/*
 * Seeded tensor generator shared by definition (not by code) with the product's model zoo: element i of
 * stream `stream` under `seed` is a pure function of (seed, stream, i), so C, C++ and numpy agree bit for bit.
 *   bits   = splitmix64(seed * 0x9E3779B97F4A7C15 + stream * 0xD1B54A32D192ED03 + 2*i [+1])
 *   u      = (bits >> 11 + 0.5) * 2^-53                 in (0,1)
 *   normal = sqrt(-2 ln u1) * cos(2 pi u2)              Box-Muller, evaluated in double
 *   value  = (float)(normal * std)     or   (float)(lo + (hi-lo) * u1) for the uniform kind
 */
static inline uint64_t orc_splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline double orc_u01(uint64_t seed, uint64_t stream, uint64_t idx) {
    uint64_t key = seed * 0x9E3779B97F4A7C15ull + stream * 0xD1B54A32D192ED03ull + idx;
    uint64_t bits = orc_splitmix64(key);
    return ((double)(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

void orc_fill_normal(float* out, size_t n, uint64_t seed, uint64_t stream, double std) {
    const double two_pi = 6.283185307179586476925286766559;
    for (size_t i = 0; i < n; ++i) {
        double u1 = orc_u01(seed, stream, 2 * i);
        double u2 = orc_u01(seed, stream, 2 * i + 1);
        double r = sqrt(-2.0 * log(u1));
        double z = r * cos(two_pi * u2);
        out[i] = (float)(z * std);
    }
}

void orc_fill_uniform(float* out, size_t n, uint64_t seed, uint64_t stream, double lo, double hi) {
    for (size_t i = 0; i < n; ++i) {
        double u1 = orc_u01(seed, stream, 2 * i);
        out[i] = (float)(lo + (hi - lo) * u1);
    }
}

/* Number of threads the OpenMP loops above will use (reported as `cores` of the CPU baseline). */
#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
#else
int orc_num_threads(void) { return 1; }
#endif
