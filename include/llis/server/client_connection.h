#pragma once
// What the server keeps per registered client: its completion ring and its wake-up socket address
// (reference include/llis/server/client_connection.h:10-37).

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>

namespace llis {
namespace server {

class ClientConnection {
  public:
    explicit ClientConnection(ClientId client_id) : client_id_(client_id) {}

    void use_s2c_channel(ipc::ShmChannelCpuWriter&& channel) { s2c_channel_ = std::move(channel); }
    void use_s2c_socket(ipc::UnixDatagramSocket&& sock) { s2c_socket_ = std::move(sock); }

    ipc::ShmChannelCpuWriter* get_s2c_channel() { return &s2c_channel_; }
    ipc::UnixDatagramSocket* get_s2c_socket() { return &s2c_socket_; }
    ClientId get_client_id() const { return client_id_; }

    // Wake-ups that could not be delivered yet because the client's socket queue was full.
    unsigned owed_wakeups = 0;

  private:
    ClientId client_id_;
    ipc::ShmChannelCpuWriter s2c_channel_;
    ipc::UnixDatagramSocket s2c_socket_;
};

}  // namespace server
}  // namespace llis
