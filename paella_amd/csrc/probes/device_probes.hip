// Device measurement probes (include/paella_probes.h): a library of its own that only the bench and the tests load; nothing
// on the serving path depends on it.

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <chrono>
#include <vector>

#include "paella_ops.h"
#include "paella_probes.h"

namespace {

__global__ void empty_kernel() {}

// Register-resident fp32 MFMA loop: four independent accumulator chains per wave, no memory traffic.
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256) void mfma_peak_kernel(float* sink, int iters) {
    probe_f32x16 acc0 = {0}, acc1 = {0}, acc2 = {0}, acc3 = {0};
    float a = 1.0f + threadIdx.x * 1e-6f, b = 1.0f - threadIdx.x * 1e-6f;
    for (int i = 0; i < iters; ++i) {
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, a, acc2, 0, 0, 0);
        acc3 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, b, acc3, 0, 0, 0);
    }
    float v = 0.f;
    for (int e = 0; e < 16; ++e) v += acc0[e] + acc1[e] + acc2[e] + acc3[e];
    if (v == 123.456f) sink[0] = v;  // keeps the loop alive without a store in practice
}

// The same loop with V independent multiply-adds after every four matrix instructions (MFMA = false: the multiply-adds alone):
// whether vector-ALU work of a SIMD's waves hides behind its matrix instructions or adds to them.
template <int V, bool MFMA>
__global__ __launch_bounds__(512) void mfma_valu_kernel(float* sink, int iters) {
    probe_f32x16 acc = {0};
    float a = 1.0f + threadIdx.x * 1e-6f, b = 1.0f - threadIdx.x * 1e-6f;
    float v[8] = {a, b, a + 1.f, b + 1.f, a + 2.f, b + 2.f, a + 3.f, b + 3.f};
    for (int i = 0; i < iters; ++i) {
        if (MFMA) {
#pragma unroll
            for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) v[j & 7] = v[j & 7] * 1.0001f + 0.5f;
        asm volatile("" ::: "memory");
    }
    float r = 0.f;
    for (int e = 0; e < 16; ++e) r += acc[e];
    for (int j = 0; j < 8; ++j) r += v[j];
    if (r == 123.456f) sink[threadIdx.x] = r;
}

template <int V, bool MFMA>
double mfma_valu_us(float* sink, int iters, unsigned blocks, hipEvent_t e0, hipEvent_t e1) {
    float best = 0.f;
    for (int rep = 0; rep < 3; ++rep) {
        hipEventRecord(e0, nullptr);
        hipLaunchKernelGGL((mfma_valu_kernel<V, MFMA>), dim3(blocks), dim3(512), 0, nullptr, sink, iters);
        hipEventRecord(e1, nullptr);
        hipEventSynchronize(e1);
        float ms = 0;
        hipEventElapsedTime(&ms, e0, e1);
        if (rep == 0 || ms < best) best = ms;
    }
    return best * 1e3;
}

}  // namespace

extern "C" {

int paella_empty_kernel_probe(int iters, double* median_us) {
    if (iters <= 0 || iters > 100000 || !median_us) return -1;
    hipStream_t st;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess) return (int)e;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    std::vector<float> us;
    for (int it = -10; it < iters; ++it) {
        // the extended launch stamps the events with the kernel's own begin and end time on the device
        hipExtLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, st, e0, e1, 0);
        hipStreamSynchronize(st);
        float ms = 0;
        if (hipEventElapsedTime(&ms, e0, e1) == hipSuccess && it >= 0) us.push_back(ms * 1e3f);
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipStreamDestroy(st);
    if (us.empty()) return -1;
    std::sort(us.begin(), us.end());
    *median_us = us[us.size() / 2];
    return 0;
}

int paella_mfma_peak_probe(double* tflops) {
    if (!tflops) return -1;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, 0);
    if (e != hipSuccess) return (int)e;
    float* sink = nullptr;
    e = hipMalloc(&sink, 64);
    if (e != hipSuccess) return (int)e;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    const int iters = 20000;
    const unsigned blocks = (unsigned)prop.multiProcessorCount * 2;  // 8 waves per CU: two per SIMD
    double best = 0;
    for (int rep = 0; rep < 3; ++rep) {
        hipEventRecord(e0, nullptr);
        hipLaunchKernelGGL(mfma_peak_kernel, dim3(blocks), dim3(256), 0, nullptr, sink, iters);
        hipEventRecord(e1, nullptr);
        hipEventSynchronize(e1);
        float ms = 0;
        hipEventElapsedTime(&ms, e0, e1);
        const double flops = (double)blocks * 4 /*waves*/ * iters * 4 /*mfma*/ * 4096.0;
        if (ms > 0 && flops / (ms * 1e-3) / 1e12 > best) best = flops / (ms * 1e-3) / 1e12;
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(sink);
    *tflops = best;
    return 0;
}

int paella_mfma_valu_overlap_probe(int valu_per_four_mfma, double* us_both, double* us_valu_alone, double* tflops) {
    if (!us_both || !us_valu_alone || !tflops) return -1;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, 0);
    if (e != hipSuccess) return (int)e;
    float* sink = nullptr;
    e = hipMalloc(&sink, 4096);
    if (e != hipSuccess) return (int)e;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    const int iters = 2000;
    const unsigned blocks = (unsigned)prop.multiProcessorCount * 4;  // 32 waves per CU: eight per SIMD
    int rc = 0;
    switch (valu_per_four_mfma) {
#define PAELLA_PROBE_CASE(V) \
    case V: *us_both = mfma_valu_us<V, true>(sink, iters, blocks, e0, e1); *us_valu_alone = mfma_valu_us<V, false>(sink, iters, blocks, e0, e1); break;
        PAELLA_PROBE_CASE(0) PAELLA_PROBE_CASE(8) PAELLA_PROBE_CASE(16) PAELLA_PROBE_CASE(32) PAELLA_PROBE_CASE(64) PAELLA_PROBE_CASE(128)
#undef PAELLA_PROBE_CASE
        default: rc = -1;
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(sink);
    if (rc == 0) *tflops = (double)blocks * 8 /*waves*/ * iters * 4 /*mfma*/ * 4096.0 / (*us_both * 1e-6) / 1e12;
    return rc;
}

int paella_queue_concurrency_probe(const paella_conv_desc* desc, int instances, int per_launch, int queues, int ordered, int reps,
                                   double* us_per_conv) {
    if (!desc || !us_per_conv || instances < 1 || instances > 64 || per_launch < 1 || per_launch > PAELLA_CONV_GROUP_MAX ||
        instances % per_launch != 0 || queues < 1 || queues > 16 || reps < 1)
        return -1;
    paella_conv_plan plan;
    if (int rc = paella_conv2d_plan(desc, 0, 0, &plan)) return rc;
    if (plan.kind != 0 || plan.mi != 1 || plan.ni != 1) return -2;
    const paella_conv_desc& d = *desc;
    std::vector<float> w((size_t)d.K * d.C * d.R * d.S);
    unsigned state = 12345u;
    for (float& v : w) {
        state = state * 1664525u + 1013904223u;
        v = ((int)(state >> 16) % 2001 - 1000) * 5e-5f;
    }
    std::vector<char> blob(plan.blob_bytes);
    if (int rc = paella_conv2d_pack(&plan, w.data(), blob.data())) return rc;
    struct Instance { void *x = nullptr, *y = nullptr, *ws = nullptr; };
    std::vector<Instance> inst((size_t)instances);
    std::vector<void*> qs;
    void *blob_dev = nullptr, *bias = nullptr;
    const size_t xb = (size_t)d.C * d.H * d.W * 4, yb = (size_t)d.K * plan.P * plan.Q * 4;
    int rc = 0;
    auto ok = [&](hipError_t e) { if (e != hipSuccess && rc == 0) rc = (int)e; return e == hipSuccess; };
    ok(hipMalloc(&blob_dev, plan.blob_bytes)) && ok(hipMemcpy(blob_dev, blob.data(), plan.blob_bytes, hipMemcpyHostToDevice));
    ok(hipMalloc(&bias, (size_t)d.K * 4)) && ok(hipMemset(bias, 0, (size_t)d.K * 4));
    for (Instance& in : inst) {
        ok(hipMalloc(&in.x, xb)) && ok(hipMemset(in.x, 0, xb));
        ok(hipMalloc(&in.y, yb));
        if (plan.workspace_bytes) ok(hipMalloc(&in.ws, plan.workspace_bytes)) && ok(hipMemset(in.ws, 0, plan.workspace_bytes));
    }
    ok(hipDeviceSynchronize());
    for (int i = 0; i < queues && rc == 0; ++i) {
        void* q = nullptr;
        rc = paella_direct_queue_create(&q);
        if (rc == 0) {
            qs.push_back(q);
            paella_direct_queue_set_ordered(q, ordered);
        }
    }
    double us = 0;
    for (int pass = 0; pass < 2 && rc == 0; ++pass) {  // a short pass first: the argument rings and the caches are warm afterwards
        const int n = pass ? reps : std::max(1, reps / 10);
        const auto t0 = std::chrono::steady_clock::now();
        for (int r = 0; r < n && rc == 0; ++r) {
            size_t qi = 0;
            for (int i = 0; i < instances && rc == 0; i += per_launch) {
                if (per_launch == 1) {
                    rc = paella_conv2d_launch(&plan, (const float*)inst[i].x, blob_dev, (const float*)bias, nullptr, nullptr, (float*)inst[i].y, inst[i].ws,
                                              qs[qi], 0, nullptr);
                } else {
                    paella_conv_operands m[PAELLA_CONV_GROUP_MAX];
                    for (int k = 0; k < per_launch; ++k)
                        m[k] = paella_conv_operands{&plan, (const float*)inst[i + k].x, blob_dev, (const float*)bias, nullptr, nullptr, (float*)inst[i + k].y,
                                                    inst[i + k].ws};
                    rc = paella_conv2d_launch_group(m, per_launch, qs[qi], 0, nullptr);
                }
                qi = (qi + 1) % qs.size();
            }
        }
        for (void* q : qs) paella_direct_queue_wait(q);
        us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / ((double)n * instances);
    }
    for (void* q : qs) paella_direct_queue_destroy(q);
    for (Instance& in : inst) {
        hipFree(in.x);
        hipFree(in.y);
        if (in.ws) hipFree(in.ws);
    }
    hipFree(blob_dev);
    hipFree(bias);
    *us_per_conv = us;
    return rc;
}

}  // extern "C"
