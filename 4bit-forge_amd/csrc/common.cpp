#include "common.h"

namespace forge {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace forge

extern "C" int forge_hip_abi_version(void) { return 1; }
extern "C" const char* forge_last_error(void) { return forge::error_buffer(); }
