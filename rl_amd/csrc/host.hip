// Host-side plumbing shared by every entry point: the per-thread error text and launch checks.

#include <cstring>

#include "common.hpp"

namespace nrl {

char* error_slot() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_slot(), 512, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(NRL_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return NRL_OK;
}

}  // namespace nrl

extern "C" int nrl_version(void) { return 111; }

extern "C" const char* nrl_last_error(void) { return nrl::error_slot(); }
