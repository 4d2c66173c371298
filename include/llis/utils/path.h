#pragma once
#include <string>

namespace llis {
namespace utils {

// Joins path components with '/', dropping duplicate separators
// (contract of reference include/llis/utils/path.h:25-28).
inline std::string path_concat(const std::string& a) { return a; }

template <typename... Rest>
inline std::string path_concat(const std::string& a, const Rest&... rest) {
    std::string tail = path_concat(std::string(rest)...);
    if (a.empty()) return tail;
    if (tail.empty()) return a;
    if (tail.front() == '/') return tail;  // an absolute component restarts the path, as std::filesystem does
    return a.back() == '/' ? a + tail : a + "/" + tail;
}

}  // namespace utils
}  // namespace llis
