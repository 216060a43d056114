// Library-wide pieces of the C ABI: version, per-thread error string.
#include <cstdarg>
#include <cstdio>

#include "common.hpp"

namespace a4g {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return A4G_OK;
    return fail(A4G_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace a4g

extern "C" int a4g_version(void) { return A4G_VERSION; }

extern "C" const char* a4g_last_error(void) { return a4g::g_error; }
