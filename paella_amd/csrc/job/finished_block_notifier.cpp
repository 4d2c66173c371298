// Host-side allocation of the device-resident notifier array, one notifier per stream of the pool
// (reference src/job/finished_block_notifier.cu:21-46).

#include <llis/job/finished_block_notifier.h>
#include <llis/utils/error.h>

#include "paella_hip.h"

#include <cstdlib>
#include <cstring>
#include <new>
#include <stdexcept>

namespace llis {
namespace job {

FinishedBlockNotifier* FinishedBlockNotifier::create_array(unsigned num, ipc::Gpu2SchedChannel* gpu2sched_channel,
                                                           ipc::Gpu2SchedChannel* block_time_channel, unsigned batch_size) {
    if (!valid_batch_size(batch_size)) throw std::invalid_argument("notification batch size must be a power of two between 1 and 128");
    const size_t bytes = (size_t)num * sizeof(FinishedBlockNotifier);
    // Build the host image in raw storage: the objects are views (non-owning), so the image can be copied
    // bit for bit to the device and dropped without running destructors.
    void* raw = std::aligned_alloc(alignof(FinishedBlockNotifier), bytes);  // sizeof is a multiple of the alignment
    if (!raw) throw std::bad_alloc();
    for (unsigned i = 0; i < num; ++i) new (reinterpret_cast<FinishedBlockNotifier*>(raw) + i) FinishedBlockNotifier(gpu2sched_channel, block_time_channel, batch_size);
    void* dev = nullptr;
    int rc = llis_hip_device_malloc(&dev, bytes);
    if (rc == 0) rc = llis_hip_memcpy(dev, raw, bytes, LLIS_HIP_H2D);
    std::free(raw);
    LLIS_CHECK_HIP(rc);
    return reinterpret_cast<FinishedBlockNotifier*>(dev);
}

void FinishedBlockNotifier::free_array(FinishedBlockNotifier* ptr) {
    if (ptr) LLIS_WARN_HIP(llis_hip_device_free(ptr));
}

}  // namespace job
}  // namespace llis
