#pragma once
// The 8-byte message a workgroup sends to the scheduler.  Bit layout (little endian, one ring slot):
//   byte 0  is_start   1 = workgroups became resident, 0 = workgroups finished, 2 = a copy stage finished
//   byte 1  smid       compute-unit id of the sender (un-aggregated hooks only)
//   byte 2  num        how many workgroups this message accounts for (1..batch size of the sending notifier, at most 128; 16 in the reference)
//   byte 3  status     1 = slot holds an unread message, 0 = consumed
//   byte 4-7 job_id
// Layout and accessor names follow reference include/llis/job/instrument_info.h:9-38; the value 2 of
// is_start is an addition used by the ring-marker path for memory stages.

#include <llis/ipc/defs.h>
#include <llis/utils/gpu.h>

#include <cstdint>

namespace llis {
namespace job {

class InstrumentInfo {
  public:
    uint8_t is_start;
    uint8_t smid;
    uint8_t num;

  private:
    uint8_t status_;

  public:
    JobId job_id;

    LLIS_HOSTDEV InstrumentInfo() : is_start(0), smid(0), num(0), status_(1), job_id(0) {}

    LLIS_HOSTDEV bool can_read() const { return status_ == 1; }
    LLIS_HOSTDEV bool can_write() const { return status_ == 0; }
    LLIS_HOSTDEV void set_can_read() { status_ = 1; }
    LLIS_HOSTDEV void set_can_write() { status_ = 0; }
};

static_assert(sizeof(InstrumentInfo) == 8, "InstrumentInfo must be exactly one 64-bit ring slot");

// Optional per-workgroup timing sample (two 24-bit clock values), same slot discipline
// (reference include/llis/job/instrument_info.h:42-70).
class BlockStartEndTime {
  private:
    uint8_t status_;
    uint8_t reserved_;

  public:
    uint16_t data[3];

    LLIS_HOSTDEV BlockStartEndTime() : status_(1), reserved_(0), data{0, 0, 0} {}

    LLIS_HOSTDEV bool can_read() const { return status_ == 1; }
    LLIS_HOSTDEV bool can_write() const { return status_ == 0; }
    LLIS_HOSTDEV void set_can_read() { status_ = 1; }
    LLIS_HOSTDEV void set_can_write() { status_ = 0; }
};

static_assert(sizeof(BlockStartEndTime) == 8, "BlockStartEndTime must be exactly one 64-bit ring slot");

}  // namespace job
}  // namespace llis
