// Error reporting and version of the C ABI.
#include "common.hpp"

namespace sgnn {

std::string &last_error() {
    static thread_local std::string msg;
    return msg;
}

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

}  // namespace sgnn

extern "C" const char *sgnn_last_error(void) { return sgnn::last_error().c_str(); }

extern "C" int sgnn_version(void) { return 1; }
