#pragma once
// Test-and-set spin lock that lives inside a shared mapping (one byte, zero = free).  Serialises whole
// messages of several producers on one byte ring (role of reference include/llis/ipc/atomic_lock.h:11-27).

#include <llis/utils/gpu.h>

namespace llis {
namespace ipc {

class AtomicLock {
  public:
    LLIS_HOSTDEV void init() { release(); }

    LLIS_HOSTDEV void acquire() {
#if defined(__HIP_DEVICE_COMPILE__)
        while (__hip_atomic_exchange(&held_, (unsigned char)1, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM)) {
        }
#else
        while (__atomic_exchange_n(&held_, (unsigned char)1, __ATOMIC_ACQUIRE)) {
#if defined(__x86_64__)
            __builtin_ia32_pause();
#endif
        }
#endif
    }

    LLIS_HOSTDEV void release() {
#if defined(__HIP_DEVICE_COMPILE__)
        __hip_atomic_store(&held_, (unsigned char)0, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
#else
        __atomic_store_n(&held_, (unsigned char)0, __ATOMIC_RELEASE);
#endif
    }

  private:
    unsigned char held_;
};

static_assert(sizeof(AtomicLock) == 1, "the lock occupies exactly one byte of the ring header");

}  // namespace ipc
}  // namespace llis
