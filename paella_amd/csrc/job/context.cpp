#include <llis/job/context.h>

namespace llis {
namespace job {

Job* Context::current_job_ = nullptr;
bool Context::stage_by_stage_ = false;
ipc::Gpu2SchedChannel Context::gpu2sched_channel_;
ipc::Gpu2SchedChannel Context::gpu2sched_block_time_channel_;
ipc::ShmChannelCpuWriter Context::mem2sched_channel_;
Context::PollHook Context::poll_hooks_[Context::kMaxPollHooks] = {};
unsigned Context::num_poll_hooks_ = 0;

void Context::add_poll_hook(PollHook fn) {
    if (!fn) return;
    for (unsigned i = 0; i < num_poll_hooks_; ++i)
        if (poll_hooks_[i] == fn) return;
    if (num_poll_hooks_ < kMaxPollHooks) poll_hooks_[num_poll_hooks_++] = fn;
}

}  // namespace job
}  // namespace llis
