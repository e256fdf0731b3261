// Error reporting shared by every entry point of the C ABI.
#include "common.h"

#include <cstdlib>

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

bool test_hooks_enabled(const char* hook) {
    static const bool on = [] {
        const char* e = std::getenv("LLMOPS_TEST_HOOKS");
        return e != nullptr && e[0] == '1' && e[1] == '\0';
    }();
    if (on) return true;
    fail(LLMOPS_EINVAL, "%s: test hooks are switched off (start the process with LLMOPS_TEST_HOOKS=1)", hook);
    static bool said = false;
    if (!said) {
        said = true;
        std::fprintf(stderr, "llmops: %s\n", last_error().c_str());
    }
    return false;
}

}  // namespace llmops

extern "C" const char* llmops_last_error(void) { return llmops::last_error().c_str(); }
extern "C" int llmops_abi_version(void) { return 1; }
