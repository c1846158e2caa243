#pragma once
#include <cstdint>
#include <memory>
#include <vector>

#include "device.h"

namespace mrk {
int create_builtin_program(int device_id, ffi::Stream stream, const char* kind, const int64_t* params, size_t nparams,
                           std::unique_ptr<Program>* out);
// COPY plan items (tensor/src/realize.rs:1002-1011: buffer-to-buffer transfers need no kernel).
// The one buffer of the item is the device side; `host` is the host side and is kept alive by
// the program.  to_device: host -> buffers[0]; otherwise buffers[0] -> host.  Queued with
// hipMemcpyAsync on the program's stream, in order with the plan's kernels.
int create_copy_program(int device_id, ffi::Stream stream, bool to_device, std::shared_ptr<std::vector<uint8_t>> host,
                        std::unique_ptr<Program>* out);
}
