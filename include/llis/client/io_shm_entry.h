#pragma once
#include <cstddef>

namespace llis {
namespace client {

// One request slot of a job type's shared-memory pool: `ptr` in this process; (id, offset) names the same
// bytes to the server as "chunk id of the pool, byte offset inside the chunk"
// (reference include/llis/client/io_shm_entry.h:15-19).
struct IoShmEntry {
    void* ptr;
    int id;
    size_t offset;
};

}  // namespace client
}  // namespace llis
