// Error convention of the C-ABI: every entry point returns an int status (0 = ok) and
// leaves a thread-local message retrievable with mrk_hip_last_error().
// Status values mirror the variants of morok's device error enum
// (device/src/error.rs:5-51): SizeMismatch, CopyFailed, InvalidDevice, NotAllocated,
// NotCpuAccessible, InvalidView, Runtime, plus a backend variant carrying the hipError_t
// name (the counterpart of CudaError{source}, error.rs:47-50).
#pragma once
#include <string>

namespace mrk {

enum Status : int {
    kOk = 0,
    kSizeMismatch = 1,
    kCopyFailed = 2,
    kInvalidDevice = 3,
    kNotAllocated = 4,
    kNotCpuAccessible = 5,
    kInvalidView = 6,
    kRuntime = 7,
    kHipError = 8,
    kRenderError = 9,
    kCompileError = 10,
    kInvalidArgument = 11,
    kTimeout = 12,
    kUnsupportedDevice = 13,
};

// Records `msg` as the calling thread's last error and returns `code`.
int fail(Status code, const std::string& msg);
// printf-style helper.
int failf(Status code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Maps a hipError_t-like integer from the FFI layer to kHipError with the error's name.
int fail_hip(int hip_code, const char* what);
const char* last_error();
// Status of the most recent fail*() on this thread since clear_error() (0 if none).
int last_status();
void clear_error();

}  // namespace mrk

// Early-return helpers used throughout the host code.
#define MRK_TRY(expr)                 \
    do {                              \
        int _mrk_rc = (expr);         \
        if (_mrk_rc != 0) return _mrk_rc; \
    } while (0)
#define MRK_HIP(expr, what)                                  \
    do {                                                     \
        int _mrk_h = (expr);                                 \
        if (_mrk_h != 0) return ::mrk::fail_hip(_mrk_h, what); \
    } while (0)
