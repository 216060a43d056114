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

// A window of rows copied on the device with the runtime's own 2-D copy (a memcpy node under stream capture).
extern "C" int a4g_copy_2d(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, int64_t rows, int64_t row_bytes,
                           a4g_stream_t stream) {
    using namespace a4g;
    const char* who = "a4g_copy_2d";
    A4G_REQUIRE(rows >= 0 && row_bytes >= 0 && ld_src >= row_bytes && ld_dst >= row_bytes, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad window rows=%lld row_bytes=%lld ld_src=%lld ld_dst=%lld", who, (long long)rows, (long long)row_bytes,
                (long long)ld_src, (long long)ld_dst);
    if (rows == 0 || row_bytes == 0) return A4G_OK;
    A4G_REQUIRE(src && dst, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    return check_hip(hipMemcpy2DAsync(dst, static_cast<size_t>(ld_dst), src, static_cast<size_t>(ld_src), static_cast<size_t>(row_bytes),
                                      static_cast<size_t>(rows), hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)), who);
}
