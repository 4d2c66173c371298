// Stand-alone exercisers and latency probes for the GPU->host notification ring (see include/paella_ring.h).

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <new>
#include <vector>

#include "direct_dispatch.h"
#include "paella_hip.h"
#include "paella_ops.h"
#include "paella_ring.h"
#include <llis/ipc/shm_primitive_channel.h>
#include <llis/job/finished_block_notifier.h>
#include <llis/job/instrument.h>

using llis::ipc::Gpu2SchedChannel;
using llis::job::FinishedBlockNotifier;
using llis::job::InstrumentInfo;

struct paella_ring {
    Gpu2SchedChannel channel;
    FinishedBlockNotifier* notifiers = nullptr;
    unsigned num_notifiers = 0;
    float* scratch = nullptr;
    size_t scratch_len = 0;
};

namespace {

__global__ void probe_agg_kernel(float* buf, unsigned count, llis::JobId job_id, FinishedBlockNotifier* notifier) {
    notifier->start(job_id);
    const unsigned nthreads = blockDim.x * gridDim.x * gridDim.y * gridDim.z;
    const unsigned block_lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    for (unsigned i = block_lin * blockDim.x + threadIdx.x; i < count; i += nthreads) buf[i] += 1.f;
    notifier->end(job_id);
}

__global__ void probe_raw_kernel(float* buf, unsigned count, llis::JobId job_id, Gpu2SchedChannel channel) {
    llis::job::kernel_start(job_id, &channel);
    const unsigned nthreads = blockDim.x * gridDim.x * gridDim.y * gridDim.z;
    const unsigned block_lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    for (unsigned i = block_lin * blockDim.x + threadIdx.x; i < count; i += nthreads) buf[i] += 1.f;
    llis::job::kernel_end(job_id, &channel);
}

// Same shape as the reference's ring latency probe: start message, grid-stride vector add, barrier, end message.
__global__ void drain_bench_kernel(float* out, const float* in, unsigned count, Gpu2SchedChannel channel) {
    if (threadIdx.x == 0) {
        InstrumentInfo info;
        info.is_start = 1;
        info.job_id = blockIdx.x;
        channel.write(info);
    }
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += blockDim.x * gridDim.x) out[i] += in[i];
    __syncthreads();
    if (threadIdx.x == 0) {
        InstrumentInfo info;
        info.is_start = 0;
        info.job_id = blockIdx.x;
        channel.write(info);
    }
}

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

__global__ void flag_kernel(int* flag) { __hip_atomic_store(flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM); }

// One lane answers `total` host pings: waits (bounded by a tick budget, and by a negative value of the flag) until
// the host has raised *go above i, reads the realtime counter, sends one ring message, keeps the counter value.
__global__ void echo_kernel(Gpu2SchedChannel channel, const int* go, unsigned long long* stamps, int total, unsigned long long budget_ticks) {
    const unsigned long long t_start = wall_clock64();
    for (int i = 0; i < total; ++i) {
        for (;;) {
            const int seen = __hip_atomic_load(go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            if (seen > i) break;
            if (seen < 0 || wall_clock64() - t_start > budget_ticks) return;
        }
        const unsigned long long g = wall_clock64();
        InstrumentInfo info;
        info.is_start = 0;
        info.num = 1;
        info.job_id = (llis::JobId)(i & 0xFFFF);
        channel.write(info);
        stamps[i] = g;
    }
}

double now_us() {
    return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

}  // namespace

extern "C" {

unsigned paella_ring_batch_size(void) { return FinishedBlockNotifier::noti_batch_size; }

int paella_ring_create(size_t slots, unsigned num_notifiers, paella_ring** out) {
    return paella_ring_create_batched(slots, num_notifiers, FinishedBlockNotifier::noti_batch_size, out);
}

int paella_ring_create_batched(size_t slots, unsigned num_notifiers, unsigned batch, paella_ring** out) {
    if (!out || slots == 0 || !FinishedBlockNotifier::valid_batch_size(batch)) return -1;
    try {
        paella_ring* r = new paella_ring();
        r->channel.connect(std::string(), slots);
        r->num_notifiers = num_notifiers;
        if (num_notifiers) r->notifiers = FinishedBlockNotifier::create_array(num_notifiers, &r->channel, nullptr, batch);
        r->scratch_len = 1u << 20;
        void* p = nullptr;
        int rc = llis_hip_device_malloc(&p, r->scratch_len * sizeof(float));
        if (rc) { delete r; return rc; }
        r->scratch = reinterpret_cast<float*>(p);
        hipMemset(r->scratch, 0, r->scratch_len * sizeof(float));
        *out = r;
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_ring_create: %s\n", e.what());
        return -1;
    }
}

int paella_ring_destroy(paella_ring* r) {
    if (!r) return -1;
    hipDeviceSynchronize();
    FinishedBlockNotifier::free_array(r->notifiers);
    if (r->scratch) llis_hip_device_free(r->scratch);
    delete r;
    return 0;
}

void* paella_ring_notifier(paella_ring* r, unsigned idx) { return (r && idx < r->num_notifiers) ? r->notifiers + idx : nullptr; }

void* paella_ring_channel(paella_ring* r) { return r ? &r->channel : nullptr; }

int paella_ring_probe_launch(paella_ring* r, unsigned notifier_idx, unsigned gx, unsigned gy, unsigned gz, unsigned block,
                             uint32_t job_id, int hooks, void* stream) {
    if (!r || gx == 0 || gy == 0 || gz == 0 || block == 0 || block > 1024) return -1;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (hooks == 0) {
        if (notifier_idx >= r->num_notifiers) return -1;
        hipLaunchKernelGGL(probe_agg_kernel, dim3(gx, gy, gz), dim3(block), 0, st, r->scratch, (unsigned)r->scratch_len, job_id,
                           r->notifiers + notifier_idx);
    } else {
        hipLaunchKernelGGL(probe_raw_kernel, dim3(gx, gy, gz), dim3(block), 0, st, r->scratch, (unsigned)r->scratch_len, job_id,
                           r->channel.fork());
    }
    return (int)hipGetLastError();
}

int paella_ring_can_read(paella_ring* r) { return r && r->channel.can_read<InstrumentInfo>() ? 1 : 0; }

size_t paella_ring_drain(paella_ring* r, uint64_t* out, size_t n, double timeout_s) {
    if (!r) return 0;
    const double deadline = now_us() + timeout_s * 1e6;
    size_t got = 0;
    unsigned spins = 0;
    while (got < n) {
        if (r->channel.can_read<InstrumentInfo>()) {
            InstrumentInfo info = r->channel.read<InstrumentInfo>();
            uint64_t bits;
            __builtin_memcpy(&bits, &info, 8);
            if (out) out[got] = bits;
            ++got;
        } else if ((++spins & 0xFFF) == 0 && now_us() > deadline) {
            break;
        }
    }
    return got;
}

int paella_ring_bench_drain(paella_ring* r, unsigned blocks, unsigned vec_len, int warmup, int iters, double* us_per_iter) {
    if (!r || blocks == 0 || iters <= 0 || !us_per_iter || (size_t)vec_len * 2 > r->scratch_len) return -1;
    hipStream_t st;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess) return (int)e;
    float* out = r->scratch;
    float* in = r->scratch + vec_len;
    double t0 = 0;
    for (int it = -warmup; it < iters; ++it) {
        if (it == 0) t0 = now_us();
        hipLaunchKernelGGL(drain_bench_kernel, dim3(blocks), dim3(100), 0, st, out, in, vec_len, r->channel.fork());
        if (paella_ring_drain(r, nullptr, (size_t)blocks * 2, 10.0) != (size_t)blocks * 2) {
            hipStreamDestroy(st);
            return -1;
        }
    }
    *us_per_iter = (now_us() - t0) / iters;
    hipStreamSynchronize(st);
    hipStreamDestroy(st);
    return 0;
}

int paella_ring_bench_pingpong(int warmup, int iters, double* flag_us, double* sync_us, double* flag_samples_us) {
    if (iters <= 0 || !flag_us || !sync_us) return -1;
    hipStream_t st;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess) return (int)e;
    void* p = nullptr;
    int rc = llis_hip_host_alloc_coherent(&p, 64);
    if (rc) return rc;
    int* flag = reinterpret_cast<int*>(p);

    double t0 = 0;
    for (int it = -warmup; it < iters; ++it) {
        if (it == 0) t0 = now_us();
        hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(1), 0, st);
        hipStreamSynchronize(st);
    }
    *sync_us = (now_us() - t0) / iters;

    double total = 0;
    for (int it = -warmup; it < iters; ++it) {
        __atomic_store_n(flag, 0, __ATOMIC_RELEASE);
        const double s = now_us();
        hipLaunchKernelGGL(flag_kernel, dim3(1), dim3(1), 0, st, flag);
        while (__atomic_load_n(flag, __ATOMIC_ACQUIRE) == 0) {
        }
        const double d = now_us() - s;
        if (it >= 0) {
            total += d;
            if (flag_samples_us) flag_samples_us[it] = d;
        }
    }
    *flag_us = total / iters;
    hipStreamSynchronize(st);
    hipStreamDestroy(st);
    llis_hip_host_free(flag);
    return 0;
}

int paella_ring_bench_echo(paella_ring* r, int warmup, int iters, double* round_trip_us, double* gpu_to_host_us) {
    if (!r || warmup < 0 || iters <= 0 || iters + warmup > 200000 || !round_trip_us) return -1;
    const int total = warmup + iters;
    uint64_t hz = 0;
    const bool have_clock = paella::direct_system_clock(nullptr, &hz) && hz > 0;
    hipStream_t st;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess) return (int)e;
    void* p = nullptr;
    int rc = llis_hip_host_alloc_coherent(&p, 64);
    if (rc) return rc;
    int* go = reinterpret_cast<int*>(p);
    __atomic_store_n(go, 0, __ATOMIC_RELEASE);
    unsigned long long* stamps = nullptr;
    e = hipMalloc(&stamps, sizeof(unsigned long long) * total);
    if (e != hipSuccess) {
        llis_hip_host_free(go);
        return (int)e;
    }
    std::vector<uint64_t> seen_at(total, 0);
    std::vector<double> rtt(total, 0);
    // the kernel gives up after 20 s of realtime-counter ticks (100 MHz) whatever the host does
    hipLaunchKernelGGL(echo_kernel, dim3(1), dim3(1), 0, st, r->channel.fork(), go, stamps, total, 2000000000ull);
    int done = 0;
    for (; done < total; ++done) {
        const double h0 = now_us();
        __atomic_store_n(go, done + 1, __ATOMIC_RELEASE);
        unsigned spins = 0;
        bool got = true;
        while (!r->channel.can_read<InstrumentInfo>()) {
            if ((++spins & 0xFFFF) == 0 && now_us() - h0 > 2e6) {
                got = false;
                break;
            }
        }
        if (!got) break;
        if (have_clock) paella::direct_system_clock(&seen_at[done], nullptr);
        rtt[done] = now_us() - h0;
        r->channel.read<InstrumentInfo>();
    }
    if (done < total) __atomic_store_n(go, -1, __ATOMIC_RELEASE);  // releases the kernel
    hipStreamSynchronize(st);
    std::vector<unsigned long long> g(total, 0);
    hipMemcpy(g.data(), stamps, sizeof(unsigned long long) * total, hipMemcpyDeviceToHost);
    hipFree(stamps);
    hipStreamDestroy(st);
    llis_hip_host_free(go);
    if (done < total) return -1;
    for (int i = 0; i < iters; ++i) {
        round_trip_us[i] = rtt[warmup + i];
        if (gpu_to_host_us) {
            uint64_t sys = 0;
            const bool ok = have_clock && paella::direct_device_tick_to_system(g[warmup + i], &sys);
            gpu_to_host_us[i] = ok ? ((double)seen_at[warmup + i] - (double)sys) * 1e6 / (double)hz : -1e30;
        }
    }
    return 0;
}

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
