#pragma once
// Fixed-slot multi-producer / single-consumer ring whose slots carry their own "ready" byte.
//
// for_gpu == true  (Gpu2SchedChannel): the slots live in fine-grained, system-coherent host memory
//   obtained from llis_hip_host_alloc_coherent(); GPU workgroups claim a slot with a device-scope wrapping
//   increment of a cursor that lives in device memory and publish the 64-bit message with one
//   system-scope release store.  The host consumer polls the slot at its read position.
// for_gpu == false: the same ring in POSIX shared memory ("llis:pchannel:<name>") or anonymous memory,
//   with the cursor inside the mapping.
//
// Semantics follow reference include/llis/ipc/shm_primitive_channel.h:11-68,
// shm_primitive_channel_impl.h:18-64 and src/ipc/shm_primitive_channel.cu:49-182: a message type U has
// sizeof(U) == sizeof(T) and exposes can_read()/set_can_write(); the writer never checks for a full ring;
// the reader hands the slot back by storing the message with its ready byte cleared.
//
// The object is a plain handle (pointers + counters, no std:: members) so it can be passed BY VALUE as a
// kernel argument, exactly like the reference's channels (reference jobs/helloworld/helloworld.cu:8,67).

#include <llis/utils/gpu.h>

#include <cstddef>
#include <cstdint>
#include <string>

namespace llis {
namespace ipc {

template <typename T, bool for_gpu>
class ShmPrimitiveChannelBase {
  public:
    ShmPrimitiveChannelBase() {}
    ShmPrimitiveChannelBase(std::string name, size_t count = 0) { connect(name, count); }
    ShmPrimitiveChannelBase(ShmPrimitiveChannelBase<T, for_gpu>* other) { connect(other); }
    ShmPrimitiveChannelBase(size_t count) { connect(std::string(), count); }
    ~ShmPrimitiveChannelBase() { disconnect(); }

    ShmPrimitiveChannelBase(const ShmPrimitiveChannelBase&) = delete;
    ShmPrimitiveChannelBase& operator=(const ShmPrimitiveChannelBase&) = delete;

    ShmPrimitiveChannelBase(ShmPrimitiveChannelBase&& rhs) { steal(rhs); }
    ShmPrimitiveChannelBase& operator=(ShmPrimitiveChannelBase&& rhs) {
        if (this != &rhs) {
            disconnect();
            steal(rhs);
        }
        return *this;
    }

    // Creates (count > 0) or attaches to (count == 0, named only) a ring.
    void connect(std::string name, size_t count = 0);
    // Non-owning view of the same ring; the view starts at the other handle's read position.
    void connect(ShmPrimitiveChannelBase<T, for_gpu>* other);

    ShmPrimitiveChannelBase<T, for_gpu> fork() {
        ShmPrimitiveChannelBase<T, for_gpu> view;
        view.connect(this);
        return view;
    }

    void disconnect();
    bool is_connected() { return slots_ != nullptr; }

    size_t get_count() const { return count_; }
    T* get_slots() const { return slots_; }
    unsigned* get_cursor() const { return cursor_; }

    template <typename U>
    LLIS_HOSTDEV U read();
    template <typename U>
    LLIS_HOSTDEV void write(U val);
    // Same, but the message store carries no release of its own: for producers that have already ordered
    // their data before the message by other means.
    template <typename U>
    LLIS_HOSTDEV void write_relaxed(U val);
    template <typename U>
    LLIS_HOSTDEV bool can_read();

  private:
    void steal(ShmPrimitiveChannelBase& rhs) {
        slots_ = rhs.slots_;
        cursor_ = rhs.cursor_;
        count_ = rhs.count_;
        read_pos_ = rhs.read_pos_;
        head_ = rhs.head_;
        base_ = rhs.base_;
        mapped_bytes_ = rhs.mapped_bytes_;
        fd_ = rhs.fd_;
        owner_ = rhs.owner_;
        for (size_t i = 0; i < sizeof(name_); ++i) name_[i] = rhs.name_[i];
        rhs.slots_ = nullptr;
        rhs.owner_ = false;
    }

    T* slots_ = nullptr;          // ring storage (host-coherent for the GPU flavour)
    unsigned* cursor_ = nullptr;  // next slot to claim; device memory for the GPU flavour
    unsigned count_ = 0;
    unsigned read_pos_ = 0;       // consumer-private
    T head_ = 0;                  // last value loaded from slots_[read_pos_]

    char* base_ = nullptr;        // start of the mapping / allocation
    size_t mapped_bytes_ = 0;
    int fd_ = -1;
    bool owner_ = false;
    char name_[96] = {0};         // "llis:pchannel:<name>" when backed by POSIX shm
};

template <typename T>
using ShmPrimitiveChannel = ShmPrimitiveChannelBase<T, false>;
template <typename T>
using ShmPrimitiveChannelGpu = ShmPrimitiveChannelBase<T, true>;

using Gpu2SchedChannel = ShmPrimitiveChannelGpu<uint64_t>;

// ---------------------------------------------------------------------------------------------------
// Hot-path members, inline for both the host consumer and the device producers.

namespace detail {

template <typename T, typename U>
LLIS_HOSTDEV inline T to_bits(const U& v) {
    static_assert(sizeof(T) == sizeof(U), "message type must be exactly one ring slot wide");
    T bits;
    __builtin_memcpy(&bits, static_cast<const void*>(&v), sizeof(T));
    return bits;
}

template <typename U, typename T>
LLIS_HOSTDEV inline U from_bits(const T& bits) {
    static_assert(sizeof(T) == sizeof(U), "message type must be exactly one ring slot wide");
    U v;
    __builtin_memcpy(static_cast<void*>(&v), &bits, sizeof(T));
    return v;
}

// Claims the next slot index: returns the old cursor and stores (old >= last ? 0 : old + 1).
LLIS_HOSTDEV inline unsigned claim_slot(unsigned* cursor, unsigned last) {
#if defined(__HIP_DEVICE_COMPILE__)
    return atomicInc(cursor, last);
#else
    // Host producers exist only where the cursor is host-addressable (CPU rings and scripted test devices).
    unsigned old = __atomic_load_n(cursor, __ATOMIC_RELAXED);
    while (!__atomic_compare_exchange_n(cursor, &old, old >= last ? 0u : old + 1u, true, __ATOMIC_RELAXED,
                                        __ATOMIC_RELAXED)) {
    }
    return old;
#endif
}

template <typename T>
LLIS_HOSTDEV inline void publish(T* slot, T bits) {
#if defined(__HIP_DEVICE_COMPILE__)
    // One system-scope release store: everything this workgroup wrote before it (and everything it
    // observed through device-scope atomics) is visible to the host and to later kernels before the
    // consumer can see the message.
    __hip_atomic_store(slot, bits, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
#else
    __atomic_store_n(slot, bits, __ATOMIC_RELEASE);
#endif
}

template <typename T>
LLIS_HOSTDEV inline void publish_relaxed(T* slot, T bits) {
#if defined(__HIP_DEVICE_COMPILE__)
    __hip_atomic_store(slot, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#else
    __atomic_store_n(slot, bits, __ATOMIC_RELEASE);
#endif
}

template <typename T>
LLIS_HOSTDEV inline T peek(const T* slot) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __hip_atomic_load(slot, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
#else
    return __atomic_load_n(slot, __ATOMIC_ACQUIRE);
#endif
}

}  // namespace detail

template <typename T, bool for_gpu>
template <typename U>
LLIS_HOSTDEV inline void ShmPrimitiveChannelBase<T, for_gpu>::write(U val) {
    const unsigned pos = detail::claim_slot(cursor_, count_ - 1);
    detail::publish(slots_ + pos, detail::to_bits<T>(val));
}

template <typename T, bool for_gpu>
template <typename U>
LLIS_HOSTDEV inline void ShmPrimitiveChannelBase<T, for_gpu>::write_relaxed(U val) {
    const unsigned pos = detail::claim_slot(cursor_, count_ - 1);
    detail::publish_relaxed(slots_ + pos, detail::to_bits<T>(val));
}

template <typename T, bool for_gpu>
template <typename U>
LLIS_HOSTDEV inline bool ShmPrimitiveChannelBase<T, for_gpu>::can_read() {
    head_ = detail::peek(slots_ + read_pos_);
    return detail::from_bits<U>(head_).can_read();
}

template <typename T, bool for_gpu>
template <typename U>
LLIS_HOSTDEV inline U ShmPrimitiveChannelBase<T, for_gpu>::read() {
    U msg = detail::from_bits<U>(head_);
    while (!msg.can_read()) {
        head_ = detail::peek(slots_ + read_pos_);
        msg = detail::from_bits<U>(head_);
    }
    // Hand the slot back: same payload, ready byte cleared (a later can_read() on this slot is false
    // until a producer overwrites it).
    msg.set_can_write();
    head_ = detail::to_bits<T>(msg);
    detail::publish(slots_ + read_pos_, head_);
    read_pos_ = (read_pos_ + 1 == count_) ? 0 : read_pos_ + 1;
    return msg;
}

}  // namespace ipc
}  // namespace llis
