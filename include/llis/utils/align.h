#pragma once
#include <llis/utils/gpu.h>

#include <cstddef>
#include <cstdint>

namespace llis {
namespace utils {

// Smallest multiple of `align` (a power of two) that is >= pos
// (same contract as reference include/llis/utils/align.h:11-13).
LLIS_HOSTDEV constexpr size_t next_aligned_pos(size_t pos, size_t align) {
    return (pos + (align - 1)) & ~(align - 1);
}

template <typename T>
LLIS_HOSTDEV inline T* next_aligned_ptr(T* ptr, size_t align) {
    return reinterpret_cast<T*>(next_aligned_pos(reinterpret_cast<uintptr_t>(ptr), align));
}

}  // namespace utils
}  // namespace llis
