"""Direct entry points of the hand-written kernels (device buffers in, device buffers out)."""
import ctypes as C

from ._ffi import check, lib
from .device import Buffer


def _p(b):
    return C.c_void_p(b.ptr if isinstance(b, Buffer) else int(b))


def softmax_f32(x, y, rows, cols, device_id=0, variant=0):
    """Fused row softmax (Tensor::softmax, tensor/src/activation.rs:90-101), last axis."""
    check(lib.mrk_hip_softmax_f32_variant(device_id, _p(x), _p(y), rows, cols, variant))
