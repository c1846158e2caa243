#include "error.h"

#include <cstdarg>
#include <cstdio>

#include "hip_ffi.h"

namespace mrk {

static thread_local std::string g_last_error;
static thread_local int g_last_status = 0;

int fail(Status code, const std::string& msg) {
    g_last_error = msg;
    g_last_status = static_cast<int>(code);
    return static_cast<int>(code);
}

int failf(Status code, const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    g_last_status = static_cast<int>(code);
    return static_cast<int>(code);
}

int fail_hip(int hip_code, const char* what) {
    // The runtime keeps the last error per thread; drop it so that a later, unrelated
    // hipGetLastError() check does not report this failure again.
    ffi::clear_last_error();
    return failf(kHipError, "HIP error: %s failed: %s (%d)", what, ffi::error_name(hip_code), hip_code);
}

const char* last_error() { return g_last_error.c_str(); }
int last_status() { return g_last_status; }
void clear_error() {
    g_last_error.clear();
    g_last_status = 0;
}

}  // namespace mrk
