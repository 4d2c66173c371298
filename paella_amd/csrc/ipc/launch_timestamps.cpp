#include <llis/ipc/defs.h>

#include <atomic>
#include <cstdlib>

namespace llis {
namespace ipc {

namespace {

bool initial() {
#ifdef PRINT_LAUNCH_JOB_IPC_LATENCY
    return true;
#else
    const char* e = std::getenv("LLIS_PRINT_LAUNCH_JOB_IPC_LATENCY");
    return e && e[0] == '1';
#endif
}

std::atomic<int>& state() {
    static std::atomic<int> s{initial() ? 1 : 0};
    return s;
}

}  // namespace

bool launch_timestamps() { return state().load(std::memory_order_relaxed) != 0; }
void set_launch_timestamps(bool on) { state().store(on ? 1 : 0, std::memory_order_relaxed); }

}  // namespace ipc
}  // namespace llis
