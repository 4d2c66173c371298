#include <llis/client/profiler_client.h>

namespace llis {
namespace client {

void ProfilerClient::send(ProfilerMsgType sub) {
    c2s_channel_->acquire_writer_lock();
    c2s_channel_->write(MsgType::PROFILER_CMD);
    c2s_channel_->write(sub);
    c2s_channel_->release_writer_lock();
}

void ProfilerClient::save(const std::string& path) {
    c2s_channel_->acquire_writer_lock();
    c2s_channel_->write(MsgType::PROFILER_CMD);
    c2s_channel_->write(ProfilerMsgType::SAVE);
    c2s_channel_->write(path);
    c2s_channel_->release_writer_lock();
}

}  // namespace client
}  // namespace llis
