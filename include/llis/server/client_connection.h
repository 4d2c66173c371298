#pragma once
// What the server keeps per registered client: the ring its completions go to, the datagram socket it is woken on,
// and the wake-ups it is still owed (reference include/llis/server/client_connection.h:10-37 holds the first two).

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>

#include <chrono>
#include <utility>

namespace llis {
namespace server {

class ClientConnection {
  public:
    explicit ClientConnection(ClientId client_id) : client_id_(client_id) {}

    ClientId get_client_id() const { return client_id_; }

    void use_s2c_channel(ipc::ShmChannelCpuWriter&& channel) { s2c_channel_ = std::move(channel); }
    void use_s2c_socket(ipc::UnixDatagramSocket&& sock) { s2c_socket_ = std::move(sock); }
    ipc::ShmChannelCpuWriter* get_s2c_channel() { return &s2c_channel_; }
    ipc::UnixDatagramSocket* get_s2c_socket() { return &s2c_socket_; }

    // One-byte poke that gets the client out of wait().  The kernel queues only a handful of datagrams per socket, and
    // a client with many requests in flight that is slow to call wait() must not stall the serving thread: the poke
    // never blocks, and one that did not fit is owed (they are all the same byte, so order does not matter).
    // Returns true if the poke is owed rather than sent.
    bool wake() {
        if (dead_) return false;
        if (owed_wakeups_ == 0 && poke()) return false;
        ++owed_wakeups_;
        return true;
    }

    // Sends as many owed pokes as fit now; returns how many are no longer owed (sent, or written off with a peer that has
    // refused every poke for kDeadAfter: a client that exited without waiting for its requests).
    unsigned retry_wakeups() {
        unsigned settled = 0;
        while (owed_wakeups_ != 0 && poke()) {
            --owed_wakeups_;
            ++settled;
        }
        if (dead_) {
            settled += owed_wakeups_;
            owed_wakeups_ = 0;
        }
        return settled;
    }

    // A dead peer gets neither pokes nor completions (its completion ring would fill up and block the serving thread).
    bool is_dead() const { return dead_; }

    static constexpr std::chrono::milliseconds kDeadAfter{2000};

  private:
    bool poke() {
        if (dead_) return false;
        const bool byte = true;
        bool refused = false;
        if (s2c_socket_.try_write(&byte, sizeof(byte), &refused)) {
            refusing_ = false;
            return true;
        }
        if (!refused) {
            refusing_ = false;
        } else if (!refusing_) {
            refusing_ = true;
            refused_since_ = std::chrono::steady_clock::now();
        } else if (std::chrono::steady_clock::now() - refused_since_ > kDeadAfter) {
            dead_ = true;
        }
        return false;
    }

    ClientId client_id_;
    unsigned owed_wakeups_ = 0;
    bool refusing_ = false, dead_ = false;
    std::chrono::steady_clock::time_point refused_since_;
    ipc::ShmChannelCpuWriter s2c_channel_;
    ipc::UnixDatagramSocket s2c_socket_;
};

}  // namespace server
}  // namespace llis
