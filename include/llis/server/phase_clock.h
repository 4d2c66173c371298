#pragma once
// Build-time diagnostic (-DLLIS_PHASE_PROFILE): cycle counters for the phases of the serving thread, printed
// when the server is destroyed.  Compiles to nothing otherwise.

#ifdef LLIS_PHASE_PROFILE
#include <x86intrin.h>

#include <cstdio>

namespace llis {
namespace server {

struct PhaseClock {
    enum Phase { kIdle, kRing, kRequests, kLaunch, kLaunchCopy, kHooks, kCount };
    unsigned long long cycles[kCount] = {};
    unsigned long long events[kCount] = {};
    static PhaseClock& get() {
        static PhaseClock clock;
        return clock;
    }
    void report() const {
        unsigned long long total = 0;
        for (int i = 0; i < kCount; ++i) total += cycles[i];
        static const char* const names[kCount] = {"idle polls", "ring messages (excl. launches)", "client requests (excl. launches)", "run_next of kernel stages", "run_next of copy stages + markers", "poll hooks of job libraries"};
        for (int i = 0; i < kCount; ++i)
            std::fprintf(stderr, "[phase] %-34s %6.2f %%  %10llu events  %8.0f cycles/event\n", names[i], 100.0 * cycles[i] / (total ? total : 1),
                         events[i], events[i] ? (double)cycles[i] / events[i] : 0.0);
    }
};

// Charges the enclosed time to `phase`; time charged by nested scopes is subtracted from the enclosing one.
class PhaseScope {
  public:
    explicit PhaseScope(PhaseClock::Phase phase) : phase_(phase), parent_(current()), start_(__rdtsc()) { current() = this; }
    ~PhaseScope() {
        const unsigned long long spent = __rdtsc() - start_;
        PhaseClock& c = PhaseClock::get();
        c.cycles[phase_] += spent - nested_;
        ++c.events[phase_];
        if (parent_) parent_->nested_ += spent;
        current() = parent_;
    }

  private:
    static PhaseScope*& current() {
        static thread_local PhaseScope* cur = nullptr;
        return cur;
    }
    PhaseClock::Phase phase_;
    PhaseScope* parent_;
    unsigned long long start_;
    unsigned long long nested_ = 0;
};

}  // namespace server
}  // namespace llis
#define LLIS_PHASE(phase) ::llis::server::PhaseScope llis_phase_scope_(::llis::server::PhaseClock::phase)
#define LLIS_PHASE_IF(cond, a, b) ::llis::server::PhaseScope llis_phase_scope_((cond) ? ::llis::server::PhaseClock::a : ::llis::server::PhaseClock::b)
#define LLIS_PHASE_REPORT() ::llis::server::PhaseClock::get().report()
// Forget everything measured before the 600th request (instance creation, weight upload, warm-up).
#define LLIS_PHASE_WARMUP_TICK()                                     \
    do {                                                             \
        static unsigned long long seen_ = 0;                         \
        if (++seen_ == 600) {                                        \
            ::llis::server::PhaseClock& c_ = ::llis::server::PhaseClock::get(); \
            for (int i_ = 0; i_ < ::llis::server::PhaseClock::kCount; ++i_) c_.cycles[i_] = c_.events[i_] = 0; \
        }                                                            \
    } while (0)
#else
#define LLIS_PHASE_WARMUP_TICK()
#define LLIS_PHASE(phase)
#define LLIS_PHASE_IF(cond, a, b)
#define LLIS_PHASE_REPORT()
#endif
