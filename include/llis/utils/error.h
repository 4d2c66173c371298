#pragma once
// Error helpers without Boost/spdlog: failures of POSIX or HIP calls raise std::runtime_error carrying the
// call site, warnings go to stderr (contract of reference include/llis/utils/error.h:10-127).

#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>

namespace llis {
namespace utils {

[[noreturn]] inline void throw_at(const char* what, const std::string& detail, const char* file, int line) {
    throw std::runtime_error(std::string(what) + ": " + detail + " (" + file + ":" + std::to_string(line) + ")");
}

// POSIX convention: `bad` is the failure value (-1 for most calls, 0 for pointer-returning ones).
inline void check_posix(intptr_t ret, intptr_t bad, const char* file, int line) {
    if (ret == bad) throw_at("posix", std::strerror(errno), file, line);
}

inline void warn_posix(intptr_t ret, intptr_t bad, const char* file, int line) {
    if (ret == bad) std::fprintf(stderr, "[llis] warning: %s (%s:%d)\n", std::strerror(errno), file, line);
}

// Return code of the llis_hip_* C-ABI: 0 is success.
void check_hip(int code, const char* file, int line);
void warn_hip(int code, const char* file, int line);

}  // namespace utils
}  // namespace llis

#define LLIS_CHECK_POSIX(expr) ::llis::utils::check_posix((intptr_t)(expr), -1, __FILE__, __LINE__)
#define LLIS_CHECK_POSIX_PTR(expr, bad) ::llis::utils::check_posix((intptr_t)(expr), (intptr_t)(bad), __FILE__, __LINE__)
#define LLIS_WARN_POSIX(expr) ::llis::utils::warn_posix((intptr_t)(expr), -1, __FILE__, __LINE__)
#define LLIS_CHECK_HIP(expr) ::llis::utils::check_hip((expr), __FILE__, __LINE__)
#define LLIS_WARN_HIP(expr) ::llis::utils::warn_hip((expr), __FILE__, __LINE__)
