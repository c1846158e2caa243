#pragma once
#include "device.h"

namespace mrk {
int create_builtin_program(int device_id, ffi::Stream stream, const char* kind, const int64_t* params, size_t nparams,
                           std::unique_ptr<Program>* out);
}
