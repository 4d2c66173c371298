// User-mode AQL queues and the HSA loader side of direct dispatch (see direct_dispatch.h).
//
// What replaces what: the reference pays cudaLaunchKernel once per stage from its scheduler thread
// (reference jobs/tvm_mnist/tvm_mnist.cpp:41 through the TVM runtime); on this platform the equivalent HIP
// call is the dominant cost of that thread, so the model adapters submit their kernels here instead.

#include <immintrin.h>
#include "direct_dispatch.h"

#include "paella_ops.h"

#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

extern "C" {
// Embedded code objects (hsaco_blobs.cpp).
extern const char paella_hsaco_conv_begin[];
extern const char paella_hsaco_conv_end[];
extern const char paella_hsaco_misc_begin[];
extern const char paella_hsaco_misc_end[];
}

namespace paella {

int g_direct_queue_count = 0;

namespace {

constexpr uint32_t kQueuePackets = 4096;       // ring size (power of two)
constexpr uint32_t kKernargSlotBytes = 2560;   // one slot per packet index: explicit args <= 2304 + implicit block 256
constexpr size_t kImplicitBytes = 256;

struct Runtime {
    bool ok = false;
    std::string error;
    hsa_agent_t gpu{};
    hsa_agent_t cpu{};
    hsa_amd_memory_pool_t kernarg_pool{};
    hsa_amd_memory_pool_t device_pool{};  // device memory the host may map (kernel arguments next to the GPU)
    bool have_gpu = false, have_cpu = false, have_pool = false, have_device_pool = false;
    std::vector<hsa_executable_t> executables;
};

std::mutex g_mutex;
Runtime g_rt;
bool g_rt_tried = false;
std::unordered_map<const void*, DirectKernel> g_kernels;  // guarded by g_mutex; entries are never erased
std::vector<DirectQueue*> g_queues;                        // guarded by g_mutex for writes

#define HSA_TRY(call, what)                                                                  \
    do {                                                                                     \
        hsa_status_t st_ = (call);                                                           \
        if (st_ != HSA_STATUS_SUCCESS && st_ != HSA_STATUS_INFO_BREAK) {                     \
            const char* msg_ = nullptr;                                                      \
            hsa_status_string(st_, &msg_);                                                   \
            g_rt.error = std::string(what) + ": " + (msg_ ? msg_ : "unknown HSA error");     \
            return false;                                                                    \
        }                                                                                    \
    } while (0)

hsa_status_t find_agents(hsa_agent_t agent, void*) {
    hsa_device_type_t type;
    if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
    if (type == HSA_DEVICE_TYPE_GPU && !g_rt.have_gpu) {
        g_rt.gpu = agent;
        g_rt.have_gpu = true;
    } else if (type == HSA_DEVICE_TYPE_CPU && !g_rt.have_cpu) {
        g_rt.cpu = agent;
        g_rt.have_cpu = true;
    }
    return HSA_STATUS_SUCCESS;
}

hsa_status_t find_kernarg_pool(hsa_amd_memory_pool_t pool, void*) {
    hsa_amd_segment_t segment;
    if (hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_SEGMENT, &segment) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
    if (segment != HSA_AMD_SEGMENT_GLOBAL) return HSA_STATUS_SUCCESS;
    uint32_t flags = 0;
    hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_GLOBAL_FLAGS, &flags);
    bool can_alloc = false;
    hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_RUNTIME_ALLOC_ALLOWED, &can_alloc);
    if ((flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_KERNARG_INIT) && can_alloc && !g_rt.have_pool) {
        g_rt.kernarg_pool = pool;
        g_rt.have_pool = true;
    }
    return HSA_STATUS_SUCCESS;
}

hsa_status_t find_device_pool(hsa_amd_memory_pool_t pool, void*) {
    hsa_amd_segment_t segment;
    if (hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_SEGMENT, &segment) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
    if (segment != HSA_AMD_SEGMENT_GLOBAL) return HSA_STATUS_SUCCESS;
    uint32_t flags = 0;
    hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_GLOBAL_FLAGS, &flags);
    bool can_alloc = false;
    hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_RUNTIME_ALLOC_ALLOWED, &can_alloc);
    hsa_amd_memory_pool_access_t access = HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED;
    hsa_amd_agent_memory_pool_get_info(g_rt.cpu, pool, HSA_AMD_AGENT_MEMORY_POOL_INFO_ACCESS, &access);
    if ((flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_COARSE_GRAINED) && can_alloc && access != HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED &&
        !g_rt.have_device_pool) {
        g_rt.device_pool = pool;
        g_rt.have_device_pool = true;
    }
    return HSA_STATUS_SUCCESS;
}

bool load_code_object(const char* begin, const char* end, const char* what) {
    hsa_code_object_reader_t reader;
    HSA_TRY(hsa_code_object_reader_create_from_memory(begin, (size_t)(end - begin), &reader), what);
    hsa_executable_t exe;
    HSA_TRY(hsa_executable_create_alt(HSA_PROFILE_FULL, HSA_DEFAULT_FLOAT_ROUNDING_MODE_DEFAULT, nullptr, &exe), what);
    HSA_TRY(hsa_executable_load_agent_code_object(exe, g_rt.gpu, reader, nullptr, nullptr), what);
    HSA_TRY(hsa_executable_freeze(exe, nullptr), what);
    g_rt.executables.push_back(exe);
    return true;
}

bool init_runtime_locked() {
    // The HIP runtime must own the device first (it initialises HSA itself); this adds a reference.
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        g_rt.error = "no HIP device";
        return false;
    }
    HSA_TRY(hsa_init(), "hsa_init");
    HSA_TRY(hsa_iterate_agents(find_agents, nullptr), "hsa_iterate_agents");
    if (!g_rt.have_gpu || !g_rt.have_cpu) {
        g_rt.error = "no GPU agent";
        return false;
    }
    HSA_TRY(hsa_amd_agent_iterate_memory_pools(g_rt.cpu, find_kernarg_pool, nullptr), "memory pools");
    if (!g_rt.have_pool) {
        g_rt.error = "no kernarg memory pool";
        return false;
    }
    hsa_amd_agent_iterate_memory_pools(g_rt.gpu, find_device_pool, nullptr);
    if (!load_code_object(paella_hsaco_conv_begin, paella_hsaco_conv_end, "load conv code object")) return false;
    if (!load_code_object(paella_hsaco_misc_begin, paella_hsaco_misc_end, "load misc code object")) return false;
    return true;
}

bool ensure_runtime() {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_rt_tried) {
        g_rt_tried = true;
        g_rt.ok = init_runtime_locked();
    }
    return g_rt.ok;
}

void queue_error(hsa_status_t status, hsa_queue_t*, void*) {
    const char* msg = nullptr;
    hsa_status_string(status, &msg);
    std::fprintf(stderr, "[paella] direct dispatch queue error: %s\n", msg ? msg : "unknown");
    std::abort();
}

}  // namespace

struct DirectQueue {
    hsa_queue_t* queue = nullptr;
    char* kernargs = nullptr;
    uint64_t write_index = 0;  // single producer: the thread that owns the queue
    uint64_t read_seen = 0;    // read index when this thread last looked
    bool device_kernargs = false;  // kernarg ring lives in device memory, written through the PCIe aperture
    bool ordered = false;      // barrier bit on every packet: kernels run one after the other, like a stream
};

DirectQueue* direct_queue_lookup_slow(void* handle) {
    // Read without the lock: the vector only grows under the lock before g_direct_queue_count is raised, and
    // queues are destroyed only when their owner stops using them.
    for (DirectQueue* q : g_queues)
        if (q == handle) return q;
    return nullptr;
}

const DirectKernel* direct_kernel(const void* host_function) {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_kernels.find(host_function);
    if (it != g_kernels.end()) return &it->second;
    const char* name = hipKernelNameRefByPtr(host_function, nullptr);
    if (!name) {
        std::fprintf(stderr, "[paella] direct dispatch: kernel %p has no device name\n", host_function);
        std::abort();
    }
    const std::string symbol_name = std::string(name) + ".kd";
    for (hsa_executable_t exe : g_rt.executables) {
        hsa_executable_symbol_t symbol;
        if (hsa_executable_get_symbol_by_name(exe, symbol_name.c_str(), &g_rt.gpu, &symbol) != HSA_STATUS_SUCCESS) continue;
        DirectKernel k;
        uint32_t kernarg = 0, lds = 0, priv = 0;
        hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_OBJECT, &k.object);
        hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_KERNARG_SEGMENT_SIZE, &kernarg);
        hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_GROUP_SEGMENT_SIZE, &lds);
        hsa_executable_symbol_get_info(symbol, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_PRIVATE_SEGMENT_SIZE, &priv);
        k.kernarg_bytes = kernarg;
        k.static_lds = lds;
        k.private_bytes = priv;
        if (k.object == 0 || kernarg > kKernargSlotBytes || priv != 0) {
            std::fprintf(stderr, "[paella] direct dispatch: kernel %s is not dispatchable (kernarg %u, scratch %u)\n", name, kernarg, priv);
            std::abort();
        }
        return &g_kernels.emplace(host_function, k).first->second;
    }
    std::fprintf(stderr, "[paella] direct dispatch: kernel %s not found in the embedded code objects\n", name);
    std::abort();
}

// Copies whole 64-byte lines to write-combining memory (the argument ring behind the PCIe aperture) with the widest
// streaming store the host has; both pointers 64-byte aligned.
__attribute__((target("avx512f"))) static void stream_lines_512(char* dst, const char* src, size_t lines) {
    for (size_t i = 0; i < lines; ++i) _mm512_stream_si512(reinterpret_cast<__m512i*>(dst + i * 64), _mm512_load_si512(src + i * 64));
}
__attribute__((target("avx"))) static void stream_lines_256(char* dst, const char* src, size_t lines) {
    for (size_t i = 0; i < lines * 2; ++i)
        _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + i * 32), _mm256_load_si256(reinterpret_cast<const __m256i*>(src + i * 32)));
}
static void stream_lines_128(char* dst, const char* src, size_t lines) {
    for (size_t i = 0; i < lines * 4; ++i)
        _mm_stream_si128(reinterpret_cast<__m128i*>(dst + i * 16), _mm_load_si128(reinterpret_cast<const __m128i*>(src + i * 16)));
}
void stream_lines(char* dst, const char* src, size_t lines) {
    static const int width = __builtin_cpu_supports("avx512f") ? 512 : __builtin_cpu_supports("avx") ? 256 : 128;
    if (width == 512) stream_lines_512(dst, src, lines);
    else if (width == 256) stream_lines_256(dst, src, lines);
    else stream_lines_128(dst, src, lines);
}

bool direct_queue_ordered(const DirectQueue* q) { return q->ordered; }

void direct_dispatch(DirectQueue* q, const DirectKernel* kernel, dim3 grid, dim3 block, unsigned dynamic_lds, const void* explicit_args,
                     size_t explicit_bytes, size_t used_bytes) {
    hsa_queue_t* hq = q->queue;
    const uint64_t index = q->write_index;
    // Ring full: wait for the packet processor (it drains without any action from this thread).
    // (The read index is a line the device writes: it is looked at again only when the copy kept here says the ring is full.)
    if (index - q->read_seen >= hq->size) {
        while (index - (q->read_seen = hsa_queue_load_read_index_scacquire(hq)) >= hq->size) {
        }
    }
    const uint32_t slot = (uint32_t)(index & (hq->size - 1));

    // Kernel arguments: explicit block, then the implicit block the compiler appends (block counts, workgroup
    // size, remainders, global offsets, number of grid dimensions, dynamic LDS size); everything else zero.
    char* ka = q->kernargs + (size_t)slot * kKernargSlotBytes;
    // The implicit block starts at the next 8-byte boundary; a kernel that uses none of it has a shorter segment.
    const size_t implicit_at = (explicit_bytes + 7) & ~(size_t)7;
    static_assert(kMaxExplicitArgBytes + kImplicitBytes <= kKernargSlotBytes, "a slot holds the largest argument block");
    if (explicit_bytes > kernel->kernarg_bytes) {
        std::fprintf(stderr, "[paella] direct dispatch: %zu argument bytes for a kernel that takes %u\n", explicit_bytes, kernel->kernarg_bytes);
        std::abort();
    }
    // The block is put together in cached memory and goes out in whole 64-byte lines, in ascending order, with streaming
    // stores: written in pieces, a line leaves the core's write-combining buffers as several partial transactions
    // (host time of the 51 launches of an Inception-v3 pass, argument ring warm: 36.5 us in pieces, 28.7 us this way).
    alignas(64) char stage[kKernargSlotBytes];
    if (used_bytes == 0 || used_bytes > explicit_bytes) used_bytes = explicit_bytes;
    std::memcpy(stage, explicit_args, used_bytes);
    struct Implicit {
        uint32_t block_count[3];
        uint16_t group_size[3];
        uint16_t remainder[3];
        uint8_t reserved0[16];
        uint64_t global_offset[3];
        uint16_t grid_dims;
        uint8_t reserved1[54];
        uint32_t dynamic_lds;
        uint8_t reserved2[132];
    };
    static_assert(sizeof(Implicit) == kImplicitBytes, "implicit kernel argument block is 256 bytes");
    static_assert(offsetof(Implicit, global_offset) == 40 && offsetof(Implicit, grid_dims) == 64 && offsetof(Implicit, dynamic_lds) == 120, "layout");
    size_t total = explicit_bytes;
    if (kernel->kernarg_bytes > implicit_at) {
        std::memset(stage + explicit_bytes, 0, implicit_at - explicit_bytes);
        Implicit imp;
        std::memset(&imp, 0, sizeof(imp));
        imp.block_count[0] = grid.x;
        imp.block_count[1] = grid.y;
        imp.block_count[2] = grid.z;
        imp.group_size[0] = (uint16_t)block.x;
        imp.group_size[1] = (uint16_t)block.y;
        imp.group_size[2] = (uint16_t)block.z;
        imp.grid_dims = grid.z > 1 ? 3 : (grid.y > 1 ? 2 : 1);
        imp.dynamic_lds = dynamic_lds;
        const size_t n = kernel->kernarg_bytes - implicit_at;
        std::memcpy(stage + implicit_at, &imp, sizeof(imp));
        total = implicit_at + (n < sizeof(imp) ? n : sizeof(imp));
    }
    if (q->device_kernargs) {
        const size_t lines = (total + 63) / 64;
        std::memset(stage + total, 0, lines * 64 - total);  // the tail of the last line is padding inside the slot
        // lines that hold neither used explicit arguments nor the implicit block stay as they are in the ring
        const size_t used_lines = (used_bytes + 63) / 64, implicit_line = total > explicit_bytes ? implicit_at / 64 : lines;
        if (implicit_line > used_lines) {
            stream_lines(ka, stage, used_lines);
            stream_lines(ka + implicit_line * 64, stage + implicit_line * 64, lines - implicit_line);
        } else {
            stream_lines(ka, stage, lines);
        }
    } else {
        std::memcpy(ka, stage, total);
    }

    if (q->device_kernargs) __builtin_ia32_sfence();  // write-combined stores out before the doorbell
    auto* pkt = reinterpret_cast<hsa_kernel_dispatch_packet_t*>(hq->base_address) + slot;
    pkt->workgroup_size_x = (uint16_t)block.x;
    pkt->workgroup_size_y = (uint16_t)block.y;
    pkt->workgroup_size_z = (uint16_t)block.z;
    pkt->reserved0 = 0;
    pkt->grid_size_x = grid.x * block.x;
    pkt->grid_size_y = grid.y * block.y;
    pkt->grid_size_z = grid.z * block.z;
    pkt->private_segment_size = 0;
    pkt->group_segment_size = kernel->static_lds + dynamic_lds;
    pkt->kernel_object = kernel->object;
    pkt->kernarg_address = ka;
    pkt->reserved2 = 0;
    pkt->completion_signal.handle = 0;
    // Header and setup share the packet's first 32 bits and are published last, with release semantics.
    // Acquire at agent scope: a kernel must not see stale lines of buffers that earlier kernels (on other XCDs)
    // or copies rewrote.  No release: operator kernels write their results through to memory and report
    // completion themselves, before the packet retires.
    constexpr int acq = HSA_FENCE_SCOPE_AGENT;
    constexpr int rel = HSA_FENCE_SCOPE_NONE;
    const uint16_t header = (uint16_t)((HSA_PACKET_TYPE_KERNEL_DISPATCH << HSA_PACKET_HEADER_TYPE) |
                                       (acq << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) |
                                       (rel << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE) |
                                       ((q->ordered ? 1 : 0) << HSA_PACKET_HEADER_BARRIER));
    const uint16_t setup = (uint16_t)(3 << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS);
    __atomic_store_n(reinterpret_cast<uint32_t*>(pkt), (uint32_t)header | ((uint32_t)setup << 16), __ATOMIC_RELEASE);

    q->write_index = index + 1;
    hsa_queue_store_write_index_screlease(hq, index + 1);
    hsa_signal_store_screlease(hq->doorbell_signal, (hsa_signal_value_t)index);
}

bool direct_system_clock(uint64_t* now_ticks, uint64_t* ticks_per_second) {
    if (!ensure_runtime()) return false;
    if (now_ticks && hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP, now_ticks) != HSA_STATUS_SUCCESS) return false;
    if (ticks_per_second && hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, ticks_per_second) != HSA_STATUS_SUCCESS) return false;
    return true;
}

bool direct_device_tick_to_system(uint64_t device_tick, uint64_t* system_tick) {
    if (!ensure_runtime() || !system_tick) return false;
    return hsa_amd_profiling_convert_tick_to_system_domain(g_rt.gpu, device_tick, system_tick) == HSA_STATUS_SUCCESS;
}

}  // namespace paella

namespace paella {
static std::vector<void*> g_shared_queues;  // the process-wide set of paella_direct_queue_shared
static std::mutex g_shared_mutex;
static std::atomic<size_t> g_shared_count{0};

uint64_t direct_shared_min_waiting() {
    // No lock: the set is filled once, under the lock, before its size is published, and never changes afterwards.
    if (g_shared_count.load(std::memory_order_acquire) == 0) return 0;
    uint64_t least = ~0ull;
    for (void* h : g_shared_queues) {
        DirectQueue* q = static_cast<DirectQueue*>(h);
        const uint64_t waiting = q->write_index - hsa_queue_load_read_index_relaxed(q->queue);
        if (waiting < least) least = waiting;
    }
    return least;
}
}  // namespace paella

// ---- C-ABI --------------------------------------------------------------------------------------

using paella::DirectQueue;

extern "C" int paella_direct_queue_create(void** out) {
    if (!out) return PAELLA_EINVAL;
    *out = nullptr;
    if (!paella::ensure_runtime()) {
        std::fprintf(stderr, "[paella] direct dispatch unavailable: %s\n", paella::g_rt.error.c_str());
        return PAELLA_ENOSUP;
    }
    auto* q = new DirectQueue();
    hsa_status_t st = hsa_queue_create(paella::g_rt.gpu, paella::kQueuePackets, HSA_QUEUE_TYPE_SINGLE, paella::queue_error, nullptr, UINT32_MAX, UINT32_MAX,
                                       &q->queue);
    if (st != HSA_STATUS_SUCCESS) {
        delete q;
        return PAELLA_ENOSUP;
    }
    void* ka = nullptr;
    const size_t ka_bytes = (size_t)q->queue->size * paella::kKernargSlotBytes;
    st = HSA_STATUS_ERROR;
    // Kernel arguments in device memory (written by the host through the PCIe aperture): every wave of a kernel
    // reads them, and fetching them from host memory instead costs about 10 us per kernel on an idle GPU.
    if (paella::g_rt.have_device_pool) {
        st = hsa_amd_memory_pool_allocate(paella::g_rt.device_pool, ka_bytes, 0, &ka);
        if (st == HSA_STATUS_SUCCESS) st = hsa_amd_agents_allow_access(1, &paella::g_rt.cpu, nullptr, ka);
        if (st != HSA_STATUS_SUCCESS && ka) {
            hsa_amd_memory_pool_free(ka);
            ka = nullptr;
        }
        if (st == HSA_STATUS_SUCCESS) {
            q->device_kernargs = true;
            // Touch every page of the ring now: the first store to a page of the aperture takes a fault (1600 against 400
            // cycles per launch until the ring has wrapped once).
            alignas(64) static const char zeros[64] = {0};
            for (size_t off = 0; off < ka_bytes; off += 64) paella::stream_lines(reinterpret_cast<char*>(ka) + off, zeros, 1);
            __builtin_ia32_sfence();
        }
    }
    if (st != HSA_STATUS_SUCCESS) {
        st = hsa_amd_memory_pool_allocate(paella::g_rt.kernarg_pool, ka_bytes, 0, &ka);
        if (st == HSA_STATUS_SUCCESS) st = hsa_amd_agents_allow_access(1, &paella::g_rt.gpu, nullptr, ka);
    }
    if (st != HSA_STATUS_SUCCESS) {
        if (ka) hsa_amd_memory_pool_free(ka);
        hsa_queue_destroy(q->queue);
        delete q;
        return PAELLA_ENOSUP;
    }
    q->kernargs = reinterpret_cast<char*>(ka);
    q->write_index = hsa_queue_load_write_index_relaxed(q->queue);
    {
        std::lock_guard<std::mutex> lock(paella::g_mutex);
        paella::g_queues.reserve(256);  // lookups iterate without the lock: never reallocate under them
        if (paella::g_queues.size() >= 256) {
            hsa_amd_memory_pool_free(ka);
            hsa_queue_destroy(q->queue);
            delete q;
            return PAELLA_ENOSUP;
        }
        paella::g_queues.push_back(q);
        __atomic_store_n(&paella::g_direct_queue_count, (int)paella::g_queues.size(), __ATOMIC_RELEASE);
    }
    *out = q;
    return 0;
}

extern "C" int paella_direct_queue_shared(void** out) {
    // A small process-wide set of unordered queues handed out round-robin: callers whose dependent work is
    // ordered by notifications (the model job adapters on the serving thread) spread their kernels over them.
    std::vector<void*>& shared = paella::g_shared_queues;
    static size_t next = 0;
    static bool failed = false;
    if (!out) return PAELLA_EINVAL;
    std::lock_guard<std::mutex> lock(paella::g_shared_mutex);
    if (shared.empty() && !failed) {
        const char* env = std::getenv("PAELLA_DIRECT_QUEUES");
        long n = env ? std::strtol(env, nullptr, 10) : 4;
        if (n < 1) n = 1;
        if (n > 32) n = 32;
        for (long i = 0; i < n; ++i) {
            void* q = nullptr;
            if (paella_direct_queue_create(&q) != 0) break;
            shared.push_back(q);
        }
        failed = shared.empty();
        paella::g_shared_count.store(shared.size(), std::memory_order_release);
    }
    if (shared.empty()) {
        *out = nullptr;
        return PAELLA_ENOSUP;
    }
    // Least-loaded first: a queue runs its kernels one at a time, so a packet placed behind a long kernel waits
    // while another queue may be empty.  Ties go round-robin.
    size_t best = next;
    uint64_t best_pending = ~0ull;
    for (size_t i = 0; i < shared.size(); ++i) {
        const size_t idx = (next + i) % shared.size();
        DirectQueue* q = static_cast<DirectQueue*>(shared[idx]);
        const uint64_t pending = q->write_index - hsa_queue_load_read_index_relaxed(q->queue);
        if (pending < best_pending) {
            best_pending = pending;
            best = idx;
            if (pending == 0) break;
        }
    }
    *out = shared[best];
    next = (best + 1) % shared.size();
    return 0;
}

extern "C" int paella_direct_queue_set_ordered(void* queue, int ordered) {
    DirectQueue* q = paella::direct_queue_lookup(queue);
    if (!q) return PAELLA_EINVAL;
    q->ordered = ordered != 0;
    return 0;
}

extern "C" int paella_direct_queue_wait(void* queue) {
    DirectQueue* q = paella::direct_queue_lookup(queue);
    if (!q) return PAELLA_EINVAL;
    // The read index passes a packet once the packet processor has launched it, not when its kernel has
    // finished: a barrier packet with a completion signal closes the gap.
    hsa_signal_t done;
    if (hsa_signal_create(1, 0, nullptr, &done) != HSA_STATUS_SUCCESS) return PAELLA_ENOSUP;
    hsa_queue_t* hq = q->queue;
    const uint64_t index = q->write_index;
    while (index - hsa_queue_load_read_index_scacquire(hq) >= hq->size) {
    }
    auto* pkt = reinterpret_cast<hsa_barrier_and_packet_t*>(hq->base_address) + (index & (hq->size - 1));
    std::memset(reinterpret_cast<char*>(pkt) + 4, 0, sizeof(*pkt) - 4);
    pkt->completion_signal = done;
    const uint16_t header = (uint16_t)((HSA_PACKET_TYPE_BARRIER_AND << HSA_PACKET_HEADER_TYPE) | (1 << HSA_PACKET_HEADER_BARRIER) |
                                       (HSA_FENCE_SCOPE_SYSTEM << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) |
                                       (HSA_FENCE_SCOPE_SYSTEM << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE));
    __atomic_store_n(reinterpret_cast<uint32_t*>(pkt), (uint32_t)header, __ATOMIC_RELEASE);
    q->write_index = index + 1;
    hsa_queue_store_write_index_screlease(hq, index + 1);
    hsa_signal_store_screlease(hq->doorbell_signal, (hsa_signal_value_t)index);
    // Bounded wait (10 s): a kernel that never finishes must not hang the caller for ever.
    const hsa_signal_value_t v = hsa_signal_wait_scacquire(done, HSA_SIGNAL_CONDITION_LT, 1, 10ull * 1000 * 1000 * 1000, HSA_WAIT_STATE_ACTIVE);
    hsa_signal_destroy(done);
    return v < 1 ? 0 : PAELLA_ETIMEDOUT;
}

extern "C" int paella_direct_queue_destroy(void* queue) {
    DirectQueue* q = paella::direct_queue_lookup(queue);
    if (!q) return PAELLA_EINVAL;
    paella_direct_queue_wait(queue);
    {
        std::lock_guard<std::mutex> lock(paella::g_mutex);
        for (auto& slot : paella::g_queues)
            if (slot == q) slot = paella::g_queues.back();
        paella::g_queues.pop_back();
        __atomic_store_n(&paella::g_direct_queue_count, (int)paella::g_queues.size(), __ATOMIC_RELEASE);
    }
    hsa_queue_destroy(q->queue);
    hsa_amd_memory_pool_free(q->kernargs);
    delete q;
    return 0;
}
