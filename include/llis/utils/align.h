#pragma once
// Rounding positions and pointers up to a power-of-two boundary (request slots in the client pool, ring headers).
#include <llis/utils/gpu.h>

#include <cstddef>
#include <cstdint>

namespace llis {
namespace utils {

// Smallest multiple of `boundary` (a power of two) that is not below `pos`; same contract as
// reference include/llis/utils/align.h:11-13.
LLIS_HOSTDEV constexpr size_t next_aligned_pos(size_t pos, size_t boundary) {
    const size_t mask = boundary - 1;
    return (pos + mask) & ~mask;
}

static_assert(next_aligned_pos(0, 8) == 0 && next_aligned_pos(1, 8) == 8 && next_aligned_pos(8, 8) == 8 && next_aligned_pos(602113, 256) == 602368,
              "next_aligned_pos rounds up to the boundary");

// The same for an address.
template <typename T>
LLIS_HOSTDEV inline T* next_aligned_ptr(T* ptr, size_t boundary) {
    const uintptr_t address = reinterpret_cast<uintptr_t>(ptr);
    return reinterpret_cast<T*>(next_aligned_pos(address, boundary));
}

}  // namespace utils
}  // namespace llis
