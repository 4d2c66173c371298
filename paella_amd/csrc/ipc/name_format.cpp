#include <llis/ipc/name_format.h>

namespace llis {
namespace ipc {

std::string s2c_socket_name(const std::string& server_name, ClientId client_id) {
    std::string s("llis-socket-s2c-");
    s += server_name;
    s += '-';
    s += std::to_string(client_id);
    return s;
}

std::string s2c_channel_name(const std::string& server_name, ClientId client_id) {
    std::string s("s2c:");
    s += server_name;
    s += ':';
    s += std::to_string(client_id);
    return s;
}

std::string c2s_channel_name(const std::string& server_name) { return std::string("c2s:") + server_name; }

}  // namespace ipc
}  // namespace llis
