// TEST DOUBLE for the llis_hip_* C-ABI (include/paella_hip.h): a scripted "device" living in host memory,
// so that the real server, schedulers, rings and client library can be driven on a machine without a GPU.
// It is built as tests/fake_device/lib/libllis_hip.so and is only ever loaded by tests.
//
// Device model: every stream is a FIFO of operations (kernel of n workgroups, ring marker, host
// callback, copy).  An operation executes when the test says so (fake_hip_step*) or, with
// FAKE_HIP_AUTORUN=1, on a background thread that always runs the oldest issued operation that is at the
// head of its stream.  Executing a kernel means posting exactly the messages the aggregated workgroup hooks
// post: ceil(n/B) start messages then ceil(n/B) end messages (full batches of B = noti_batch_size first, remainder last);
// a raw-hook kernel (fake_hip_raw_kernel_launch) posts one start and one end message per workgroup with a compute-unit id.

#include "paella_hip.h"

#include <llis/job/context.h>
#include <llis/job/finished_block_notifier.h>
#include <llis/job/instrument_info.h>

#include <unistd.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

namespace {

enum OpKind { OP_KERNEL, OP_MARKER, OP_HOSTFUNC, OP_COPY };

struct Op {
    OpKind kind;
    uint64_t seq;
    uint32_t job_id = 0;
    unsigned nblocks = 0;
    bool raw = false;       // kernel with un-aggregated hooks: one message per workgroup, naming a compute unit
    unsigned first_xcd = 0; // raw kernels: XCD of workgroup 0
    int phase = 0;  // kernels: 0 = not started, 1 = start messages posted
    uint64_t message = 0;
    uint64_t* slots = nullptr;
    unsigned count = 0;
    unsigned* cursor = nullptr;
    void (*fn)(void*) = nullptr;
    void* arg = nullptr;
};

struct Stream {
    std::deque<Op> q;
};

// Leaked on purpose: the autorun thread may still be running while static destructors execute at exit.
std::mutex& g_mtx = *new std::mutex();
std::vector<Stream*>& g_streams = *new std::vector<Stream*>();
uint64_t g_seq = 0;
std::atomic<bool> g_autorun_started{false};
std::atomic<unsigned long long> g_ops_executed{0};

void post(uint8_t is_start, unsigned num, uint32_t job_id) {
    llis::job::InstrumentInfo info;
    info.is_start = is_start;
    info.num = (uint8_t)num;
    info.job_id = job_id;
    llis::job::Context::get_gpu2sched_channel()->write(info);
}

unsigned g_batch = llis::job::FinishedBlockNotifier::noti_batch_size;

// Where the scripted device runs workgroup i of a raw-hook kernel: XCDs take turns from where the last raw kernel stopped
// (as on the real part); inside the XCD a fixed scatter that knows nothing of what is resident -- so an occupancy model's
// predictions hold for the XCD and often miss the compute unit.
unsigned g_raw_next_xcd = 0;

unsigned raw_cu(const struct Op& op, unsigned i);

void post_raw(uint8_t is_start, const struct Op& op);

void post_batches(uint8_t is_start, unsigned n, uint32_t job_id) {
    const unsigned B = g_batch;
    for (unsigned i = 0; i < n / B; ++i) post(is_start, B, job_id);
    if (n % B) post(is_start, n % B, job_id);
}

unsigned raw_cu(const Op& op, unsigned i) {
    const unsigned xcd = (op.first_xcd + i) % 8;
    const unsigned in_xcd = (i / 8 * 5 + (unsigned)(op.seq % 7) * 3) % 32;
    return xcd * 32 + in_xcd;
}

void post_raw(uint8_t is_start, const Op& op) {
    for (unsigned i = 0; i < op.nblocks; ++i) {
        llis::job::InstrumentInfo info;
        info.is_start = is_start;
        info.smid = (uint8_t)raw_cu(op, i);
        info.num = 1;
        info.job_id = op.job_id;
        llis::job::Context::get_gpu2sched_channel()->write(info);
    }
}

// Advances the head operation of `s` by one phase (full = run it to completion).  Caller holds g_mtx,
// which is dropped around host callbacks.
bool advance(Stream* s, bool full, std::unique_lock<std::mutex>& lk) {
    if (s->q.empty()) return false;
    Op& op = s->q.front();
    switch (op.kind) {
        case OP_KERNEL:
            if (op.phase == 0) {
                if (op.raw) {
                    op.first_xcd = g_raw_next_xcd;
                    g_raw_next_xcd = (g_raw_next_xcd + op.nblocks) % 8;
                    post_raw(1, op);
                } else {
                    post_batches(1, op.nblocks, op.job_id);
                }
                op.phase = 1;
                if (!full) return true;
            }
            if (op.raw) post_raw(0, op);
            else post_batches(0, op.nblocks, op.job_id);
            break;
        case OP_MARKER: {
            unsigned old = __atomic_load_n(op.cursor, __ATOMIC_RELAXED);
            while (!__atomic_compare_exchange_n(op.cursor, &old, old >= op.count - 1 ? 0u : old + 1u, true, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {
            }
            __atomic_store_n(op.slots + old, op.message, __ATOMIC_RELEASE);
            break;
        }
        case OP_HOSTFUNC: {
            Op copy = op;
            s->q.pop_front();
            lk.unlock();
            copy.fn(copy.arg);
            lk.lock();
            ++g_ops_executed;
            return true;
        }
        case OP_COPY:
            break;
    }
    s->q.pop_front();
    ++g_ops_executed;
    return true;
}

Stream* oldest_stream() {
    Stream* best = nullptr;
    for (Stream* s : g_streams)
        if (s && !s->q.empty() && (!best || s->q.front().seq < best->q.front().seq)) best = s;
    return best;
}

void autorun_loop() {
    const char* us = std::getenv("FAKE_HIP_OP_US");
    const unsigned delay = us ? (unsigned)std::atoi(us) : 0;
    for (;;) {
        bool did = false;
        {
            std::unique_lock<std::mutex> lk(g_mtx);
            if (Stream* s = oldest_stream()) did = advance(s, true, lk);
        }
        if (!did) usleep(20);
        else if (delay) usleep(delay);
    }
}

void maybe_start_autorun() {
    const char* env = std::getenv("FAKE_HIP_AUTORUN");
    if (env && *env == '1' && !g_autorun_started.exchange(true)) std::thread(autorun_loop).detach();
}

void enqueue(void* stream, Op op) {
    std::lock_guard<std::mutex> lk(g_mtx);
    op.seq = g_seq++;
    reinterpret_cast<Stream*>(stream)->q.push_back(op);
}

}  // namespace

extern "C" {

// ---- control surface for tests and fake job definitions
// Workgroups per aggregated message of the scripted kernels (what the notifiers of a real device are created with).
void fake_hip_set_batch(unsigned batch) { g_batch = batch ? batch : llis::job::FinishedBlockNotifier::noti_batch_size; }

int fake_hip_kernel_launch(void* stream, uint32_t job_id, unsigned nblocks) {
    Op op{OP_KERNEL, 0};
    op.job_id = job_id;
    op.nblocks = nblocks;
    enqueue(stream, op);
    return 0;
}

// A kernel whose workgroups report one by one through the un-aggregated hooks.
int fake_hip_raw_kernel_launch(void* stream, uint32_t job_id, unsigned nblocks) {
    Op op{OP_KERNEL, 0};
    op.job_id = job_id;
    op.nblocks = nblocks;
    op.raw = true;
    enqueue(stream, op);
    return 0;
}

// Runs the oldest issued operation that heads its stream; returns 1 if something ran.
int fake_hip_step_oldest(int full) {
    std::unique_lock<std::mutex> lk(g_mtx);
    Stream* s = oldest_stream();
    return s ? (int)advance(s, full != 0, lk) : 0;
}

// Advances the head operation of stream number `index` (creation order).
int fake_hip_step_stream(unsigned index, int full) {
    std::unique_lock<std::mutex> lk(g_mtx);
    if (index >= g_streams.size() || !g_streams[index]) return 0;
    return (int)advance(g_streams[index], full != 0, lk);
}

unsigned long long fake_hip_ops_executed(void) { return g_ops_executed.load(); }

unsigned fake_hip_pending(void) {
    std::lock_guard<std::mutex> lk(g_mtx);
    unsigned n = 0;
    for (Stream* s : g_streams)
        if (s) n += (unsigned)s->q.size();
    return n;
}

// ---- the llis_hip_* ABI
int llis_hip_device_count(int* count) { *count = 1; return 0; }
int llis_hip_set_device(int) { return 0; }

int llis_hip_get_device_caps(llis_hip_device_caps* caps) {
    std::memset(caps, 0, sizeof(*caps));
    caps->num_cus = 256;
    caps->wavefront_size = 64;
    caps->max_threads_per_cu = 2048;
    caps->max_blocks_per_cu = 32;
    caps->vgprs_per_cu = 131072;
    caps->lds_bytes_per_cu = 163840;
    caps->clock_khz = 2400000;
    caps->l2_bytes = 4 << 20;
    std::snprintf(caps->name, sizeof(caps->name), "fake-gfx950");
    return 0;
}

const char* llis_hip_error_string(int code) { return code == 0 ? "success" : "fake device error"; }

int llis_hip_stream_create(void** stream) {
    maybe_start_autorun();
    std::lock_guard<std::mutex> lk(g_mtx);
    Stream* s = new Stream();
    g_streams.push_back(s);
    *stream = s;
    return 0;
}

int llis_hip_stream_destroy(void* stream) {
    std::lock_guard<std::mutex> lk(g_mtx);
    for (Stream*& s : g_streams)
        if (s == stream) s = nullptr;
    delete reinterpret_cast<Stream*>(stream);
    return 0;
}

int llis_hip_stream_synchronize(void*) { return 0; }
int llis_hip_stream_busy(void* stream) {
    std::lock_guard<std::mutex> lk(g_mtx);
    return reinterpret_cast<Stream*>(stream)->q.empty() ? 0 : 1;
}
int llis_hip_device_synchronize(void) { return 0; }

int llis_hip_device_malloc(void** ptr, size_t bytes) { *ptr = std::calloc(1, bytes ? bytes : 1); return *ptr ? 0 : 2; }
int llis_hip_device_free(void* ptr) { std::free(ptr); return 0; }
int llis_hip_host_alloc_coherent(void** ptr, size_t bytes) { return posix_memalign(ptr, 4096, bytes ? bytes : 1) ? 2 : (std::memset(*ptr, 0, bytes), 0); }
int llis_hip_host_alloc_pinned(void** ptr, size_t bytes) { return llis_hip_host_alloc_coherent(ptr, bytes); }
int llis_hip_host_free(void* ptr) { std::free(ptr); return 0; }

int llis_hip_memcpy(void* dst, const void* src, size_t bytes, int) { std::memcpy(dst, src, bytes); return 0; }

int llis_hip_memcpy_async(void* dst, const void* src, size_t bytes, int, void* stream) {
    std::memcpy(dst, src, bytes);  // data moves at issue time; completion is what the stream orders
    Op op{OP_COPY, 0};
    enqueue(stream, op);
    return 0;
}

int llis_hip_fill_u32_async(void* dst, uint32_t value, size_t count, void* stream) {
    for (size_t i = 0; i < count; ++i) reinterpret_cast<uint32_t*>(dst)[i] = value;
    Op op{OP_COPY, 0};
    enqueue(stream, op);
    return 0;
}

int llis_hip_launch_host_func(void* stream, void (*fn)(void*), void* arg) {
    Op op{OP_HOSTFUNC, 0};
    op.fn = fn;
    op.arg = arg;
    enqueue(stream, op);
    return 0;
}

int llis_hip_launch_ring_marker(void* stream, uint64_t* slots, unsigned count, unsigned* cursor, uint64_t message) {
    Op op{OP_MARKER, 0};
    op.slots = slots;
    op.count = count;
    op.cursor = cursor;
    op.message = message;
    enqueue(stream, op);
    return 0;
}

int llis_hip_event_create(void** event) { *event = std::malloc(8); return 0; }
int llis_hip_event_destroy(void* event) { std::free(event); return 0; }
int llis_hip_event_record(void*, void*) { return 0; }
int llis_hip_event_synchronize(void*) { return 0; }
int llis_hip_event_elapsed_ms(void*, void*, float* ms) { *ms = 0; return 0; }
int llis_hip_profiler_start(void) { return 0; }
int llis_hip_profiler_stop(void) { return 0; }

}  // extern "C"
