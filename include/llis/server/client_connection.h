#pragma once
// What the server keeps per registered client: the ring its completions go to, the datagram socket it is woken on,
// and the wake-ups it is still owed (reference include/llis/server/client_connection.h:10-37 holds the first two).

#include <llis/ipc/defs.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>

#include <chrono>
#include <cstdio>
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
        if (owed_wakeups_ == 0 && poke()) return false;
        ++owed_wakeups_;
        return true;
    }

    // Sends as many owed pokes as fit now; returns how many are no longer owed.
    unsigned retry_wakeups() {
        unsigned settled = 0;
        while (owed_wakeups_ != 0 && poke()) {
            --owed_wakeups_;
            ++settled;
        }
        return settled;
    }

    // A peer that has refused every poke for kDeadAfter is taken for dead: a client that exited without waiting for its
    // requests.  Refusal alone does not prove it -- some sandboxed kernels refuse where Linux says "queue full" -- so nothing
    // is thrown away on that verdict that still has a place to go: pokes stay owed and one is tried every kProbeEvery, and the
    // first that gets through brings the connection back (both transitions are logged).
    bool is_dead() const { return dead_; }

    // Posts a completion.  To a live peer this may wait for room in its ring, as in the reference; to a dead one it never
    // waits: without room the completion is dropped, and with it one owed poke (returns 1 then, else 0 -- the server keeps
    // the sum of owed pokes over all connections).
    unsigned post_completion(void* remote_ptr) {
        if (dead_ && !s2c_channel_.has_room(sizeof(remote_ptr))) {
            ++dropped_completions_;
            if (owed_wakeups_ == 0) return 0;
            --owed_wakeups_;
            return 1;
        }
        s2c_channel_.write(remote_ptr);
        return 0;
    }

    unsigned long long dropped_completions() const { return dropped_completions_; }

    static constexpr std::chrono::milliseconds kDeadAfter{2000};
    static constexpr std::chrono::milliseconds kProbeEvery{200};

  private:
    bool poke() {
        const auto now = std::chrono::steady_clock::now;
        if (dead_) {
            const auto t = now();
            if (t - last_probe_ < kProbeEvery) return false;
            last_probe_ = t;
        }
        const bool byte = true;
        bool refused = false;
        if (s2c_socket_.try_write(&byte, sizeof(byte), &refused)) {
            refusing_ = false;
            if (dead_) {
                dead_ = false;
                std::fprintf(stderr, "[llis] client %u takes wake-ups again; %llu completions were dropped meanwhile\n", (unsigned)client_id_, dropped_completions_);
            }
            return true;
        }
        if (dead_) return false;
        if (!refused) {
            refusing_ = false;
        } else if (!refusing_) {
            refusing_ = true;
            refused_since_ = now();
        } else if (now() - refused_since_ > kDeadAfter) {
            dead_ = true;
            last_probe_ = now();
            std::fprintf(stderr, "[llis] client %u has refused every wake-up for %lld ms: taken for dead (completions only while its ring has room)\n",
                         (unsigned)client_id_, (long long)kDeadAfter.count());
        }
        return false;
    }

    ClientId client_id_;
    unsigned owed_wakeups_ = 0;
    bool refusing_ = false, dead_ = false;
    std::chrono::steady_clock::time_point refused_since_, last_probe_;
    unsigned long long dropped_completions_ = 0;
    ipc::ShmChannelCpuWriter s2c_channel_;
    ipc::UnixDatagramSocket s2c_socket_;
};

}  // namespace server
}  // namespace llis
