#pragma once
// Single-reader byte ring in shared memory, used for client->server requests ("c2s"), server->client
// completions ("s2c") and, inside the server, copy-stage completions posted by runtime callback threads.
//
// Mapping layout (part of the IPC protocol; byte offsets on LP64):
//     0  size_t   capacity of the ring in bytes (usable: capacity - 1)
//     8  size_t   read position   (written by the reader, release)
//    16  size_t   write position  (written by the writer, release)
//    24  1 byte   writer lock     (producers that share the ring hold it around a whole message)
//    25  ...      ring bytes
// A named ring is the POSIX shm object "llis:channel:<name>"; the creator passes the capacity and unlinks
// the name when it disconnects, an attacher passes 0 and learns the capacity from the header.  An unnamed
// ring is an anonymous shared mapping.  fork() returns the opposite endpoint over the same mapping.
// Both read() and write() block by spinning.  Strings travel as size_t length + bytes.
//
// Layout and semantics follow reference include/llis/ipc/shm_channel.h:17-125,
// shm_channel_impl.h:36-120 and src/ipc/shm_channel.cu:53-170, so either side of the protocol can be a
// reference-built binary.  for_gpu == true places the mapping in system-coherent host memory so a GPU
// lane can be the writer (reference tests/ipc/shm_channel/shmc_read_write_cpu_gpu.cu:5-32).

#include <llis/ipc/atomic_lock.h>
#include <llis/utils/gpu.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>

namespace llis {
namespace ipc {

template <bool for_gpu> class ShmChannelReader;
template <bool for_gpu> class ShmChannelWriter;

template <bool for_gpu>
class ShmChannelBase {
  public:
    ShmChannelBase() {}
    ShmChannelBase(const std::string& name, size_t size = 0) { connect(name, size); }
    ShmChannelBase(ShmChannelBase<for_gpu>* other) { connect(other); }
    ShmChannelBase(size_t size) { connect(std::string(), size); }
    ~ShmChannelBase() { disconnect(); }

    ShmChannelBase(const ShmChannelBase&) = delete;
    ShmChannelBase& operator=(const ShmChannelBase&) = delete;
    ShmChannelBase(ShmChannelBase&& rhs) { steal(rhs); }
    ShmChannelBase& operator=(ShmChannelBase&& rhs) {
        if (this != &rhs) {
            disconnect();
            steal(rhs);
        }
        return *this;
    }

    void connect(std::string name, size_t size = 0);
    void connect(ShmChannelBase<for_gpu>* other);
    void disconnect();
    bool is_connected() { return base_ != nullptr; }

    static constexpr size_t kReadPosOffset = 8, kWritePosOffset = 16, kLockOffset = 24, kRingOffset = 25;

  protected:
    void steal(ShmChannelBase& rhs) {
        base_ = rhs.base_;
        ring_ = rhs.ring_;
        size_ = rhs.size_;
        mapped_bytes_ = rhs.mapped_bytes_;
        read_pos_ = rhs.read_pos_;
        write_pos_ = rhs.write_pos_;
        lock_ = rhs.lock_;
        my_read_ = rhs.my_read_;
        my_write_ = rhs.my_write_;
        fd_ = rhs.fd_;
        owner_ = rhs.owner_;
        for (size_t i = 0; i < sizeof(name_); ++i) name_[i] = rhs.name_[i];
        rhs.base_ = nullptr;
        rhs.owner_ = false;
    }

    LLIS_HOSTDEV static size_t load_pos(const size_t* p) {
#if defined(__HIP_DEVICE_COMPILE__)
        return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
#else
        return __atomic_load_n(p, __ATOMIC_ACQUIRE);
#endif
    }
    LLIS_HOSTDEV static void store_pos(size_t* p, size_t v) {
#if defined(__HIP_DEVICE_COMPILE__)
        __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
#else
        __atomic_store_n(p, v, __ATOMIC_RELEASE);
#endif
    }
    LLIS_HOSTDEV static void copy_bytes(char* dst, const char* src, size_t n) {
#if defined(__HIP_DEVICE_COMPILE__)
        for (size_t i = 0; i < n; ++i) reinterpret_cast<volatile char*>(dst)[i] = src[i];
#else
        __builtin_memcpy(dst, src, n);
#endif
    }

    char* base_ = nullptr;
    char* ring_ = nullptr;
    size_t size_ = 0;
    size_t mapped_bytes_ = 0;
    size_t* read_pos_ = nullptr;   // shared
    size_t* write_pos_ = nullptr;  // shared
    AtomicLock* lock_ = nullptr;   // shared
    size_t my_read_ = 0;           // this endpoint's view
    size_t my_write_ = 0;
    int fd_ = -1;
    bool owner_ = false;
    char name_[120] = {0};
};

template <bool for_gpu>
class ShmChannelReader : public ShmChannelBase<for_gpu> {
  public:
    using ShmChannelBase<for_gpu>::ShmChannelBase;

    ShmChannelWriter<for_gpu> fork() {
        ShmChannelWriter<for_gpu> w;
        w.connect(this);
        return w;
    }

    // Blocks until `size` bytes have been consumed.
    LLIS_HOSTDEV void read(void* buf, size_t size) {
        char* out = reinterpret_cast<char*>(buf);
        while (size > 0) {
            size_t wr = this->my_write_;
            while (wr == this->my_read_) wr = this->load_pos(this->write_pos_);  // empty: wait for the writer
            this->my_write_ = wr;
            // contiguous readable span: up to the writer, or up to the end of the ring if it has wrapped
            const size_t span_end = wr > this->my_read_ ? wr : this->size_;
            size_t n = span_end - this->my_read_;
            if (n > size) n = size;
            this->copy_bytes(out, this->ring_ + this->my_read_, n);
            out += n;
            size -= n;
            this->my_read_ += n;
            if (this->my_read_ == this->size_) this->my_read_ = 0;
            this->store_pos(this->read_pos_, this->my_read_);
        }
    }

    template <typename T>
    LLIS_HOSTDEV void read(T* value) {
        read(value, sizeof(T));
    }

    void read(std::string* str) {
        size_t len;
        read(&len);
        str->resize(len);
        if (len) read(&(*str)[0], len);
    }

    template <typename T>
    void read(std::unique_ptr<T>* ptr) {
        T* raw;
        read(&raw);
        ptr->reset(raw);
    }

    LLIS_HOSTDEV bool can_read() {
        if (this->my_write_ != this->my_read_) return true;
        this->my_write_ = this->load_pos(this->write_pos_);
        return this->my_write_ != this->my_read_;
    }
};

template <bool for_gpu>
class ShmChannelWriter : public ShmChannelBase<for_gpu> {
  public:
    using ShmChannelBase<for_gpu>::ShmChannelBase;

    ShmChannelReader<for_gpu> fork() {
        ShmChannelReader<for_gpu> r;
        r.connect(this);
        return r;
    }

    // Blocks until `size` bytes have been produced (one byte of the ring always stays empty).
    LLIS_HOSTDEV void write(const void* buf, size_t size) {
        const char* in = reinterpret_cast<const char*>(buf);
        while (size > 0) {
            size_t rd = this->my_read_;
            size_t next = this->my_write_ + 1 == this->size_ ? 0 : this->my_write_ + 1;
            while (next == rd) rd = this->load_pos(this->read_pos_);  // full: wait for the reader
            this->my_read_ = rd;
            // contiguous writable span that keeps one byte free in front of the reader
            size_t n;
            if (rd > this->my_write_) {
                n = rd - this->my_write_ - 1;
            } else {
                n = this->size_ - this->my_write_ - (rd == 0 ? 1 : 0);
            }
            if (n > size) n = size;
            this->copy_bytes(this->ring_ + this->my_write_, in, n);
            in += n;
            size -= n;
            this->my_write_ += n;
            if (this->my_write_ == this->size_) this->my_write_ = 0;
            this->store_pos(this->write_pos_, this->my_write_);
        }
    }

    template <typename T>
    LLIS_HOSTDEV void write(T value) {
        write(&value, sizeof(T));
    }

    // True if write() of `size` bytes would return without waiting for the reader.
    bool has_room(size_t size) {
        this->my_read_ = this->load_pos(this->read_pos_);
        const size_t used = this->my_write_ >= this->my_read_ ? this->my_write_ - this->my_read_ : this->size_ - this->my_read_ + this->my_write_;
        return this->size_ - 1 - used >= size;
    }

    void write(const std::string& str) {
        write(str.size());
        write(str.data(), str.size());
    }

    template <typename T>
    void write(std::unique_ptr<T>&& ptr) {
        write(reinterpret_cast<uintptr_t>(ptr.release()));
    }

    // A ring shared by several producers: hold the lock around each whole message.  The lock only orders
    // producers that share THIS endpoint object's positions or re-read them (see refresh in acquire).
    LLIS_HOSTDEV void acquire_writer_lock() {
        this->lock_->acquire();
        // Another producer may have advanced the ring by any amount since this endpoint last wrote: both cached
        // positions are stale (a read position more than a lap old would overstate the free space).
        this->my_write_ = this->load_pos(this->write_pos_);
        this->my_read_ = this->load_pos(this->read_pos_);
    }
    LLIS_HOSTDEV void release_writer_lock() { this->lock_->release(); }
};

using ShmChannelCpuReader = ShmChannelReader<false>;
using ShmChannelCpuWriter = ShmChannelWriter<false>;
using ShmChannelGpuReader = ShmChannelReader<true>;
using ShmChannelGpuWriter = ShmChannelWriter<true>;

}  // namespace ipc
}  // namespace llis
