#pragma once
// AF_UNIX / SOCK_DGRAM socket in the abstract namespace (sun_path[0] == 0, name from byte 1).
// The server keeps one unbound socket and derives a "connected" handle per client that only remembers
// the destination address; a client binds its own name and blocks in read() until the server pokes it --
// the one deliberate sleep/wake point of the protocol (reference src/ipc/unix_datagram_socket.cpp:12-84).

#include <string>

#include <sys/types.h>
#include <sys/un.h>

namespace llis {
namespace ipc {

class UnixDatagramSocket {
  public:
    UnixDatagramSocket();
    explicit UnixDatagramSocket(const std::string& name);
    UnixDatagramSocket(UnixDatagramSocket&& rhs);
    UnixDatagramSocket& operator=(UnixDatagramSocket&& rhs);
    ~UnixDatagramSocket();

    UnixDatagramSocket(const UnixDatagramSocket&) = delete;
    UnixDatagramSocket& operator=(const UnixDatagramSocket&) = delete;

    void bind(const std::string& name);
    // A non-owning handle on the same descriptor whose write() goes to `name`.
    UnixDatagramSocket connect(const std::string& name);

    ssize_t write(const void* buf, size_t count);
    // Never blocks: false when the receiver's queue is full right now (the datagram was not sent).
    // *refused (optional): the failure was ECONNREFUSED -- nobody is bound to the name (any more), or, on some
    // sandboxed kernels, the queue is full.
    bool try_write(const void* buf, size_t count, bool* refused = nullptr);
    ssize_t read(void* buf, size_t count);

  private:
    UnixDatagramSocket(int fd, bool owner) : fd_(fd), owner_(owner) {}
    static void fill_address(sockaddr_un* addr, const std::string& name);
    void close_if_owned();

    int fd_ = -1;
    bool owner_ = false;
    sockaddr_un remote_{};
};

}  // namespace ipc
}  // namespace llis
