// Mapping set-up and teardown of the byte ring (hot-path members are inline in the header).

#include <llis/ipc/shm_channel.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <cerrno>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstring>
#include <stdexcept>

namespace llis {
namespace ipc {

template <bool for_gpu>
void ShmChannelBase<for_gpu>::connect(std::string name, size_t size) {
    disconnect();
    const bool named = !name.empty();
    if (!named && size == 0) throw std::invalid_argument("an anonymous byte ring needs a capacity > 0");
    if (named && for_gpu) throw std::invalid_argument("a GPU-writable byte ring cannot live in named shared memory");
    if (size == 1) throw std::invalid_argument("a byte ring of capacity 1 can hold nothing");

    owner_ = size > 0;
    name_[0] = 0;
    fd_ = -1;

    if (named) {
        std::snprintf(name_, sizeof(name_), "llis:channel:%s", name.c_str());
        if (owner_) {
            // A creator that died without unlinking leaves an object of this name behind (with whatever positions it
            // held): remove it and insist on a fresh one, so nobody attaches to the stale ring.
            if (shm_unlink(name_) != 0 && errno != ENOENT) LLIS_WARN_POSIX(-1);
            fd_ = shm_open(name_, O_CREAT | O_EXCL | O_RDWR, 0600);
        } else {
            fd_ = shm_open(name_, O_RDWR, 0600);
        }
        LLIS_CHECK_POSIX(fd_);
        if (!owner_) {
            // The creator may still be between shm_open and ftruncate: wait for a non-empty object.
            struct stat st;
            for (int spin = 0;; ++spin) {
                LLIS_CHECK_POSIX(fstat(fd_, &st));
                if ((size_t)st.st_size >= kRingOffset + 2) break;
                if (spin > 100000) throw std::runtime_error(std::string("byte ring never sized: ") + name_);
                usleep(10);
            }
            void* hdr = mmap(nullptr, sizeof(size_t), PROT_READ, MAP_SHARED, fd_, 0);
            LLIS_CHECK_POSIX_PTR(hdr, MAP_FAILED);
            size = *reinterpret_cast<volatile size_t*>(hdr);
            LLIS_WARN_POSIX(munmap(hdr, sizeof(size_t)));
        }
    }

    size_ = size;
    mapped_bytes_ = kRingOffset + size;
    if (for_gpu) {
        void* p = nullptr;
        LLIS_CHECK_HIP(llis_hip_host_alloc_coherent(&p, mapped_bytes_));
        base_ = reinterpret_cast<char*>(p);
    } else if (named) {
        if (owner_) LLIS_CHECK_POSIX(ftruncate(fd_, (off_t)mapped_bytes_));
        base_ = reinterpret_cast<char*>(mmap(nullptr, mapped_bytes_, PROT_READ | PROT_WRITE, MAP_SHARED, fd_, 0));
        LLIS_CHECK_POSIX_PTR(base_, MAP_FAILED);
    } else {
        base_ = reinterpret_cast<char*>(mmap(nullptr, mapped_bytes_, PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0));
        LLIS_CHECK_POSIX_PTR(base_, MAP_FAILED);
    }

    read_pos_ = reinterpret_cast<size_t*>(base_ + kReadPosOffset);
    write_pos_ = reinterpret_cast<size_t*>(base_ + kWritePosOffset);
    lock_ = reinterpret_cast<AtomicLock*>(base_ + kLockOffset);
    ring_ = base_ + kRingOffset;

    if (owner_) {
        store_pos(read_pos_, 0);
        store_pos(write_pos_, 0);
        lock_->init();
        __atomic_store_n(reinterpret_cast<size_t*>(base_), size, __ATOMIC_RELEASE);
        my_read_ = my_write_ = 0;
    } else {
        my_read_ = load_pos(read_pos_);
        my_write_ = load_pos(write_pos_);
    }
}

template <bool for_gpu>
void ShmChannelBase<for_gpu>::connect(ShmChannelBase<for_gpu>* other) {
    disconnect();
    base_ = other->base_;
    ring_ = other->ring_;
    size_ = other->size_;
    mapped_bytes_ = other->mapped_bytes_;
    read_pos_ = other->read_pos_;
    write_pos_ = other->write_pos_;
    lock_ = other->lock_;
    my_read_ = other->my_read_;
    my_write_ = other->my_write_;
    fd_ = -1;
    owner_ = false;
    std::memcpy(name_, other->name_, sizeof(name_));
}

template <bool for_gpu>
void ShmChannelBase<for_gpu>::disconnect() {
    if (!is_connected()) return;
    if (for_gpu) {
        if (owner_) LLIS_WARN_HIP(llis_hip_host_free(base_));
    } else if (name_[0] != 0) {
        if (fd_ != -1) {  // endpoints made by connect(other) borrow the mapping
            LLIS_WARN_POSIX(munmap(base_, mapped_bytes_));
            LLIS_WARN_POSIX(close(fd_));
            if (owner_) LLIS_WARN_POSIX(shm_unlink(name_));
        }
    } else if (owner_) {
        LLIS_WARN_POSIX(munmap(base_, mapped_bytes_));
    }
    base_ = nullptr;
    ring_ = nullptr;
    owner_ = false;
    fd_ = -1;
}

template class ShmChannelBase<false>;
template class ShmChannelBase<true>;

}  // namespace ipc
}  // namespace llis
