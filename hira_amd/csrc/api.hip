// ABI version and thread-local error text of libhira_hip.so.
#include <stdarg.h>

#include "common.hip.h"

namespace hira {

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

}  // namespace hira

extern "C" int hira_abi_version(void) { return HIRA_ABI_VERSION; }

extern "C" const char* hira_last_error(void) { return hira::error_buffer(); }
