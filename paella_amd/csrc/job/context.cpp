#include <llis/job/context.h>

namespace llis {
namespace job {

Job* Context::current_job_ = nullptr;
bool Context::stage_by_stage_ = false;
ipc::Gpu2SchedChannel Context::gpu2sched_channel_;
ipc::Gpu2SchedChannel Context::gpu2sched_block_time_channel_;
ipc::ShmChannelCpuWriter Context::mem2sched_channel_;

}  // namespace job
}  // namespace llis
