#pragma once
// Names of the per-server and per-client IPC endpoints (reference src/ipc/name_format.cpp:7-17).

#include <llis/ipc/defs.h>

#include <string>

namespace llis {
namespace ipc {

// Abstract-namespace datagram socket on which client <id> is woken: "llis-socket-s2c-<server>-<id>"
std::string s2c_socket_name(const std::string& server_name, ClientId client_id);
// Byte ring server -> client <id>: "s2c:<server>:<id>" (POSIX object "llis:channel:s2c:<server>:<id>")
std::string s2c_channel_name(const std::string& server_name, ClientId client_id);
// Byte ring all clients -> server: "c2s:<server>"
std::string c2s_channel_name(const std::string& server_name);

}  // namespace ipc
}  // namespace llis
