// Error reporting shared by every entry point of the C ABI.
#include "common.h"

namespace llmops {

std::string& last_error() {
    static thread_local std::string e;
    return e;
}

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

}  // namespace llmops

extern "C" const char* llmops_last_error(void) { return llmops::last_error().c_str(); }
extern "C" int llmops_abi_version(void) { return 1; }
