// Host-to-host copies off the calling thread: one helper thread per process copies request inputs from the client's
// shared-memory pool into the pinned staging buffers, so that the serving thread, which must keep reading the
// notification ring, is not deaf for the 20 to 40 us such a copy takes.  The helper makes no call into the GPU runtime
// (two threads inside the runtime contend for more than the copy costs); the job issues the host-to-device copy itself
// once the helper has reported.

#include "paella_ops.h"

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <mutex>
#include <thread>

#include <pthread.h>
#include <sched.h>

namespace {

struct CopyItem {
    void* dst;
    const void* src;
    size_t bytes;
    void (*done)(void*);
    void* arg;
};

class CopyWorker {
  public:
    CopyWorker() : creators_cpu_(sched_getcpu()), thread_([this] { run(); }) { thread_.detach(); }

    // False when the helper is asleep (no copy for kSpin): the caller copies by itself, as it would without a helper --
    // a wake-up through the kernel costs more than a lone request gains -- and the helper is woken for the ones that follow.
    bool submit(const CopyItem& item) {
        if (sleeping_.load(std::memory_order_acquire)) {
            {
                std::lock_guard<std::mutex> lock(mutex_);
                woken_ = true;
            }
            wake_.notify_one();
            return false;
        }
        {
            std::lock_guard<std::mutex> lock(mutex_);
            queue_.push_back(item);
        }
        pending_.fetch_add(1, std::memory_order_release);
        if (sleeping_.load(std::memory_order_acquire)) wake_.notify_one();
        return true;
    }

  private:
    // After its last copy the helper spins for this long before it goes to sleep: from a few thousand requests per second
    // on it is always awake, and below that the serving thread has time to copy by itself.
    static constexpr std::chrono::microseconds kSpin{500};

    // A thread inherits the affinity of its creator, and the creator is a serving thread that is usually pinned to one
    // core, on which it spins: the helper must not share that core.  It may run anywhere else.
    static void leave_creators_core(int creators_cpu) {
        cpu_set_t set;
        CPU_ZERO(&set);
        for (int c = 0; c < CPU_SETSIZE; ++c) CPU_SET(c, &set);
        if (creators_cpu >= 0) CPU_CLR(creators_cpu, &set);
        (void)pthread_setaffinity_np(pthread_self(), sizeof(set), &set);  // the kernel intersects with what the process may use
    }

    void run() {
        leave_creators_core(creators_cpu_);
        for (;;) {
            if (pending_.load(std::memory_order_acquire) == 0) {
                const auto t0 = std::chrono::steady_clock::now();
                while (pending_.load(std::memory_order_acquire) == 0 && std::chrono::steady_clock::now() - t0 < kSpin) __builtin_ia32_pause();
                if (pending_.load(std::memory_order_acquire) == 0) {
                    std::unique_lock<std::mutex> lock(mutex_);
                    sleeping_.store(true, std::memory_order_release);
                    woken_ = false;
                    wake_.wait(lock, [this] { return woken_ || !queue_.empty(); });
                    sleeping_.store(false, std::memory_order_release);
                }
            }
            CopyItem item;
            {
                std::lock_guard<std::mutex> lock(mutex_);
                if (queue_.empty()) continue;
                item = queue_.front();
                queue_.pop_front();
            }
            pending_.fetch_sub(1, std::memory_order_acq_rel);
            std::memcpy(item.dst, item.src, item.bytes);
            item.done(item.arg);
        }
    }

    std::mutex mutex_;
    std::condition_variable wake_;
    std::deque<CopyItem> queue_;
    std::atomic<int> pending_{0};
    std::atomic<bool> sleeping_{false};
    bool woken_ = false;  // under mutex_
    int creators_cpu_;
    std::thread thread_;  // last member: the thread starts with everything above constructed
};

}  // namespace

extern "C" int paella_host_copy_submit(void* dst, const void* src, size_t bytes, void (*done)(void*), void* arg) {
    if (!dst || !src || !done) return PAELLA_EINVAL;
    static CopyWorker* worker = new CopyWorker();  // lives until the process ends; its thread is never joined
    return worker->submit(CopyItem{dst, src, bytes, done, arg}) ? 0 : PAELLA_EBUSY;
}
