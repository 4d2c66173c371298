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

}  // extern "C"
