// Host-callable launchers of the hand-written gfx950 kernels.  Each returns the raw
// hipError_t (0 = success) of the launch; all work is queued on `stream`.
#pragma once
#include <cstddef>
#include <cstdint>

namespace mrk {

// y = softmax(x, axis=-1), x and y f32 [rows, cols] row-major.  variant 0 = default.
int launch_softmax_f32(void* stream, const void* x, void* y, long rows, long cols, int variant);

}  // namespace mrk
