// Host-side plumbing shared by every entry point: per-thread error text and launch checking.
#include "common.h"

namespace flux {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return FLUX_OK;
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return static_cast<int>(e);
}

}  // namespace flux

extern "C" int flux_abi_version(void) { return FLUX_ABI_VERSION; }
extern "C" const char* flux_last_error(void) { return flux::g_err; }
