// Allocation and teardown of the fixed-slot ring (hot-path members are inline in the header).
//
// Memory layout of a mapping:  [size_t count][cursor (CPU flavour only)] pad [T slots[count]], rounded up
// to whole pages, as in reference src/ipc/shm_primitive_channel.cu:86-95.  The GPU flavour obtains the
// mapping from llis_hip_host_alloc_coherent() (fine-grained, device-mapped host memory) and keeps its
// cursor in device memory, where the reference registers an mmap with the CUDA runtime
// (reference src/ipc/shm_primitive_channel.cu:107-124).

#include <llis/ipc/shm_primitive_channel.h>
#include <llis/utils/align.h>
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

namespace {

struct Layout {
    size_t cursor_off;
    size_t slots_off;
    size_t total;
};

template <typename T, bool for_gpu>
Layout layout_for(size_t count) {
    Layout l;
    size_t pos = sizeof(size_t);
    l.cursor_off = utils::next_aligned_pos(pos, alignof(unsigned));
    if (!for_gpu) pos = l.cursor_off + sizeof(unsigned);
    l.slots_off = utils::next_aligned_pos(pos, alignof(T) < 8 ? 8 : alignof(T));
    l.total = utils::next_aligned_pos(l.slots_off + count * sizeof(T), (size_t)sysconf(_SC_PAGE_SIZE));
    return l;
}

}  // namespace

template <typename T, bool for_gpu>
void ShmPrimitiveChannelBase<T, for_gpu>::connect(std::string name, size_t count) {
    disconnect();
    const bool named = !name.empty();
    if (named && for_gpu) throw std::invalid_argument("a GPU-writable ring cannot live in named shared memory");
    if (!named && count == 0) throw std::invalid_argument("an anonymous ring needs a slot count > 0");
    if (count > 0xFFFFFFFFull) throw std::invalid_argument("ring too large");

    owner_ = count > 0;
    name_[0] = 0;
    fd_ = -1;

    if (named) {
        std::snprintf(name_, sizeof(name_), "llis:pchannel:%s", name.c_str());
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
            void* hdr = mmap(nullptr, sizeof(size_t), PROT_READ, MAP_SHARED, fd_, 0);
            LLIS_CHECK_POSIX_PTR(hdr, MAP_FAILED);
            count = *reinterpret_cast<size_t*>(hdr);
            LLIS_WARN_POSIX(munmap(hdr, sizeof(size_t)));
        }
    }

    const Layout l = layout_for<T, for_gpu>(count);
    mapped_bytes_ = l.total;
    if (for_gpu) {
        void* p = nullptr;
        LLIS_CHECK_HIP(llis_hip_host_alloc_coherent(&p, l.total));
        base_ = reinterpret_cast<char*>(p);
        void* cur = nullptr;
        LLIS_CHECK_HIP(llis_hip_device_malloc(&cur, sizeof(unsigned)));
        cursor_ = reinterpret_cast<unsigned*>(cur);
    } else {
        if (named) {
            if (owner_) LLIS_CHECK_POSIX(ftruncate(fd_, (off_t)l.total));
            base_ = reinterpret_cast<char*>(mmap(nullptr, l.total, PROT_READ | PROT_WRITE, MAP_SHARED, fd_, 0));
        } else {
            base_ = reinterpret_cast<char*>(mmap(nullptr, l.total, PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0));
        }
        LLIS_CHECK_POSIX_PTR(base_, MAP_FAILED);
        cursor_ = reinterpret_cast<unsigned*>(base_ + l.cursor_off);
    }

    slots_ = reinterpret_cast<T*>(base_ + l.slots_off);
    count_ = (unsigned)count;
    read_pos_ = 0;
    head_ = 0;

    if (owner_) {
        std::memset(base_, 0, l.total);
        *reinterpret_cast<size_t*>(base_) = count;
        if (for_gpu) {
            const unsigned zero = 0;
            LLIS_CHECK_HIP(llis_hip_memcpy(cursor_, &zero, sizeof(zero), LLIS_HIP_H2D));
        }
    }
}

template <typename T, bool for_gpu>
void ShmPrimitiveChannelBase<T, for_gpu>::connect(ShmPrimitiveChannelBase<T, for_gpu>* other) {
    disconnect();
    slots_ = other->slots_;
    cursor_ = other->cursor_;
    count_ = other->count_;
    read_pos_ = other->read_pos_;
    head_ = 0;
    base_ = other->base_;
    mapped_bytes_ = other->mapped_bytes_;
    fd_ = -1;
    owner_ = false;
    std::memcpy(name_, other->name_, sizeof(name_));
}

template <typename T, bool for_gpu>
void ShmPrimitiveChannelBase<T, for_gpu>::disconnect() {
    if (!is_connected()) return;
    if (for_gpu) {
        if (owner_) {
            LLIS_WARN_HIP(llis_hip_device_free(cursor_));
            LLIS_WARN_HIP(llis_hip_host_free(base_));
        }
    } else if (name_[0] != 0) {
        if (fd_ != -1) {  // views created by connect(other) share the owner's mapping and must not unmap it
            LLIS_WARN_POSIX(munmap(base_, mapped_bytes_));
            LLIS_WARN_POSIX(close(fd_));
            if (owner_) LLIS_WARN_POSIX(shm_unlink(name_));
        }
    } else if (owner_) {
        LLIS_WARN_POSIX(munmap(base_, mapped_bytes_));
    }
    slots_ = nullptr;
    cursor_ = nullptr;
    base_ = nullptr;
    owner_ = false;
    fd_ = -1;
}

template class ShmPrimitiveChannelBase<uint32_t, true>;
template class ShmPrimitiveChannelBase<uint64_t, true>;
template class ShmPrimitiveChannelBase<uint8_t, false>;
template class ShmPrimitiveChannelBase<uint16_t, false>;
template class ShmPrimitiveChannelBase<uint32_t, false>;
template class ShmPrimitiveChannelBase<uint64_t, false>;

}  // namespace ipc
}  // namespace llis
