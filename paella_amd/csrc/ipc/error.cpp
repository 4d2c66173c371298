#include <llis/utils/error.h>

#include "paella_hip.h"

namespace llis {
namespace utils {

void check_hip(int code, const char* file, int line) {
    if (code != 0) throw_at("hip", std::string(llis_hip_error_string(code)) + " (" + std::to_string(code) + ")", file, line);
}

void warn_hip(int code, const char* file, int line) {
    if (code != 0) std::fprintf(stderr, "[llis] warning: hip: %s (%s:%d)\n", llis_hip_error_string(code), file, line);
}

}  // namespace utils
}  // namespace llis
