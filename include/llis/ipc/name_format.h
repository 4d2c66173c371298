#pragma once
// Names of the IPC endpoints of one server (values as in reference src/ipc/name_format.cpp:7-17; a client and a
// server must agree on them byte for byte):
//
//   requests, all clients -> server      byte ring   "c2s:<server>"               POSIX object "llis:channel:c2s:<server>"
//   completions, server -> client <id>   byte ring   "s2c:<server>:<id>"          POSIX object "llis:channel:s2c:<server>:<id>"
//   wake-up of client <id>               datagram    "llis-socket-s2c-<server>-<id>" in the abstract socket namespace
//
// During registration a client uses a temporary id of its own choosing for the reply ring, then switches to the id
// the server assigned.

#include <llis/ipc/defs.h>

#include <string>

namespace llis {
namespace ipc {

std::string c2s_channel_name(const std::string& server_name);
std::string s2c_channel_name(const std::string& server_name, ClientId client_id);
std::string s2c_socket_name(const std::string& server_name, ClientId client_id);

}  // namespace ipc
}  // namespace llis
