#include <llis/ipc/unix_datagram_socket.h>
#include <llis/utils/error.h>

#include <sys/socket.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>
#include <stdexcept>

namespace llis {
namespace ipc {

UnixDatagramSocket::UnixDatagramSocket() {
    fd_ = ::socket(AF_UNIX, SOCK_DGRAM, 0);
    LLIS_CHECK_POSIX(fd_);
    owner_ = true;
}

UnixDatagramSocket::UnixDatagramSocket(const std::string& name) : UnixDatagramSocket() { bind(name); }

UnixDatagramSocket::UnixDatagramSocket(UnixDatagramSocket&& rhs) : fd_(rhs.fd_), owner_(rhs.owner_), remote_(rhs.remote_) {
    rhs.fd_ = -1;
    rhs.owner_ = false;
}

UnixDatagramSocket& UnixDatagramSocket::operator=(UnixDatagramSocket&& rhs) {
    if (this != &rhs) {
        close_if_owned();
        fd_ = rhs.fd_;
        owner_ = rhs.owner_;
        remote_ = rhs.remote_;
        rhs.fd_ = -1;
        rhs.owner_ = false;
    }
    return *this;
}

UnixDatagramSocket::~UnixDatagramSocket() { close_if_owned(); }

void UnixDatagramSocket::close_if_owned() {
    if (owner_ && fd_ != -1) LLIS_WARN_POSIX(::close(fd_));
    fd_ = -1;
    owner_ = false;
}

void UnixDatagramSocket::fill_address(sockaddr_un* addr, const std::string& name) {
    if (name.size() > sizeof(addr->sun_path) - 2) throw std::invalid_argument("socket name too long: " + name);
    std::memset(addr, 0, sizeof(*addr));
    addr->sun_family = AF_UNIX;
    // Leading NUL selects the abstract namespace.  The whole zero-padded sun_path is the name, which is
    // what a peer that passes sizeof(sockaddr_un) expects.
    std::memcpy(addr->sun_path + 1, name.data(), name.size());
}

void UnixDatagramSocket::bind(const std::string& name) {
    sockaddr_un addr;
    fill_address(&addr, name);
    LLIS_CHECK_POSIX(::bind(fd_, reinterpret_cast<const sockaddr*>(&addr), sizeof(addr)));
}

UnixDatagramSocket UnixDatagramSocket::connect(const std::string& name) {
    UnixDatagramSocket peer(fd_, false);
    fill_address(&peer.remote_, name);
    return peer;
}

ssize_t UnixDatagramSocket::write(const void* buf, size_t count) {
    ssize_t n = ::sendto(fd_, buf, count, 0, reinterpret_cast<const sockaddr*>(&remote_), sizeof(remote_));
    LLIS_CHECK_POSIX(n);
    return n;
}

bool UnixDatagramSocket::try_write(const void* buf, size_t count, bool* refused) {
    ssize_t n = ::sendto(fd_, buf, count, MSG_DONTWAIT, reinterpret_cast<const sockaddr*>(&remote_), sizeof(remote_));
    if (refused) *refused = n < 0 && errno == ECONNREFUSED;
    if (n >= 0) return true;
    // A receiver whose queue is full reports EAGAIN on Linux; some sandboxed kernels report ECONNREFUSED, which is also
    // what a receiver that no longer exists gives: the caller tells the two apart by how long it lasts.
    if (errno == EAGAIN || errno == EWOULDBLOCK || errno == ENOBUFS || errno == ECONNREFUSED) return false;
    LLIS_CHECK_POSIX(n);
    return false;
}

ssize_t UnixDatagramSocket::read(void* buf, size_t count) {
    ssize_t n = ::read(fd_, buf, count);
    LLIS_CHECK_POSIX(n);
    return n;
}

}  // namespace ipc
}  // namespace llis
