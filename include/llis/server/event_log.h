#pragma once
// Deterministic record of everything the scheduler consumed and decided, in the order it happened.
//
// Inputs  (what a replay must be fed):
//   J <job_id> <job_type> <unique_id> <first_stage_is_mem>   a request was admitted and given a JobId
//   B <job_id> <is_start> <num> [<cu>]                     a workgroup message was read from the GPU ring; <cu> (the compute unit
//                                                          the message names) only where the scheduler uses it: per-compute-unit
//                                                          placement, stage with un-aggregated hooks
//   M <job_id>                                             a copy stage completed
//   L <job_id> <stage> <length_us as C99 hex float>        the measured length fed to the stage estimator
// Decisions (what a replay must reproduce bit for bit):
//   D <job_id> <stage> <stream_index> <notifier_index|-1> <is_mem> <unfit>   a stage was issued
//   S <job_id>                                             client woken (pre-notify)
//   E <job_id>                                             completion posted to the client
//   R <job_id> <mispredicted_workgroups> <compute_units>   per-compute-unit placement: all workgroups of the stage have reported
//                                                          where they run; so many were predicted elsewhere, on so many compute units
// The reference has no such log; it exists so that "scheduling and notification order" can be compared
// exactly against an independent replay of the policy, on scripted and on real devices.

#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

namespace llis {
namespace server {

struct Event {
    char kind;
    int64_t a, b, c, d, e;
    double x;
};

class EventLog {
  public:
    bool enabled() const { return enabled_; }
    void enable(bool on) { enabled_ = on; }
    void clear() { events_.clear(); }
    const std::vector<Event>& events() const { return events_; }

    void add(char kind, int64_t a = 0, int64_t b = 0, int64_t c = 0, int64_t d = 0, int64_t e = 0, double x = 0) {
        if (enabled_) events_.push_back(Event{kind, a, b, c, d, e, x});
    }

    std::string to_text() const;
    bool save(const std::string& path) const;

  private:
    bool enabled_ = false;
    std::vector<Event> events_;
};

}  // namespace server
}  // namespace llis
