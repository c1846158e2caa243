"""Lazy tensors on the HIP device: a thin handle over the mrk_hip_tensor_* entry points.

Method names follow morok's Tensor (tensor/src/lib.rs, data.rs, matmul.rs, activation.rs,
reduce.rs, nn/norm.rs, transformer.rs).  Every op only extends the graph held by
libmorok_hip.so; realize() / to_numpy() run it on the GPU.  bfloat16 data crosses this
boundary as uint16 bit patterns (numpy has no bfloat16).
"""
import ctypes as C

import numpy as np

from . import uop
from ._ffi import c_i64_p, check, lib
from .device import Buffer, ExecutionPlan

_NP_OF = {uop.F32: np.float32, uop.F64: np.float64, uop.F16: np.float16, uop.BF16: np.uint16, uop.I32: np.int32,
          uop.I64: np.int64, uop.U32: np.uint32, uop.U8: np.uint8, uop.I8: np.int8, uop.BOOL: np.bool_,
          uop.I16: np.int16, uop.U16: np.uint16, uop.U64: np.uint64}
_TAG_OF = {np.dtype(np.float32): uop.F32, np.dtype(np.float64): uop.F64, np.dtype(np.float16): uop.F16,
           np.dtype(np.int32): uop.I32, np.dtype(np.int64): uop.I64, np.dtype(np.uint32): uop.U32,
           np.dtype(np.uint8): uop.U8, np.dtype(np.int8): uop.I8, np.dtype(np.bool_): uop.BOOL,
           np.dtype(np.int16): uop.I16, np.dtype(np.uint64): uop.U64}


def _i64(seq):
    seq = [int(v) for v in seq]
    return (C.c_int64 * max(len(seq), 1))(*seq), len(seq)


def set_fusion(enabled):
    """Hand-written fused kernels on (default) or off for the calling thread."""
    lib.mrk_hip_tensor_set_fusion(int(bool(enabled)))


def last_kernels():
    """Entry-point names of the kernels the last realize on this thread launched."""
    return [lib.mrk_hip_tensor_last_kernel_name(i).decode() for i in range(lib.mrk_hip_tensor_last_kernel_count())]


def last_kernel_sources():
    """Rendered HIP C per kernel of the last realize ("" for hand-written kernels)."""
    return [lib.mrk_hip_tensor_last_kernel_source(i).decode() for i in range(lib.mrk_hip_tensor_last_kernel_count())]


def last_cached_count():
    return lib.mrk_hip_tensor_last_cached_count()


def last_memory_plan():
    """(buffers reused, bytes saved) by the memory planner in the last realize / prepare."""
    return lib.mrk_hip_tensor_last_buffers_reused(), lib.mrk_hip_tensor_last_memory_saved()


def last_intermediate_bytes():
    """Device bytes the intermediates of the last realize / prepare occupy (the planner's pool after
    reuse, or one block per intermediate with MOROK_NO_MEMORY_PLANNER=1)."""
    return lib.mrk_hip_tensor_last_intermediate_bytes()


def last_beam_search():
    """(candidates compiled and timed, kernels answered by the disk cache) for the generated
    elementwise / reduce kernels of the last realize / prepare under MOROK_BEAM."""
    return lib.mrk_hip_tensor_last_beam_candidates(), lib.mrk_hip_tensor_last_beam_cache_hits()


def last_elapsed_ms():
    return lib.mrk_hip_tensor_last_elapsed_ms()


class Tensor:
    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.mrk_hip_tensor_release(h)

    # ---- creation
    @classmethod
    def from_numpy(cls, arr, dtype=None, device_id=0):
        """Tensor::from_slice / from_raw_bytes.  `dtype` overrides the tag (uint16 + BF16)."""
        arr = np.ascontiguousarray(arr)
        tag = dtype if dtype is not None else _TAG_OF[arr.dtype]
        shape, nd = _i64(arr.shape)
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_from_bytes(device_id, arr.ctypes.data_as(C.c_void_p), arr.nbytes, shape, nd, tag,
                                            C.byref(h)))
        return cls(h)

    @classmethod
    def from_slice(cls, data, dtype=None):
        """Tensor::from_slice (tensor/src/data.rs:27-36): a tensor on the CPU device; its bytes stay
        in host memory until it is moved with to() and the result is realized."""
        arr = np.ascontiguousarray(data)
        if arr.dtype == np.float64 and dtype is None:
            arr = arr.astype(np.float32)  # Python floats stand for f32 literals
        tag = dtype if dtype is not None else _TAG_OF[arr.dtype]
        shape, nd = _i64(arr.shape)
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_from_host_bytes(arr.ctypes.data_as(C.c_void_p), arr.nbytes, shape, nd, tag, C.byref(h)))
        return cls(h)

    @classmethod
    def from_slice_with(cls, data, device="CPU", dtype=None):
        """Tensor::from_slice_with(..).device(..) (data.rs:39-52): host data, then to(device)."""
        return cls.from_slice(data, dtype).to(device)

    def to(self, device):
        """Tensor::to (tensor/src/lib.rs:479-486): a lazy COPY to "CPU" / "HIP:0"; the same tensor when
        it already lives there."""
        return self._new(lib.mrk_hip_tensor_to, str(device).encode())

    @property
    def device(self):
        buf = C.create_string_buffer(32)
        check(lib.mrk_hip_tensor_device(self._h, buf, 32))
        return buf.value.decode()

    @classmethod
    def from_bytes(cls, raw, shape, dtype, device_id=0):
        raw = bytes(raw)
        shp, nd = _i64(shape)
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_from_bytes(device_id, C.cast(C.c_char_p(raw), C.c_void_p), len(raw), shp, nd, dtype,
                                            C.byref(h)))
        return cls(h)

    @classmethod
    def from_buffer(cls, buf, shape, dtype):
        shp, nd = _i64(shape)
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_from_buffer(buf._h, shp, nd, dtype, C.byref(h)))
        return cls(h)

    @classmethod
    def const(cls, value, dtype=uop.F32, device_id=0):
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_const(device_id, float(value), dtype, C.byref(h)))
        return cls(h)

    @classmethod
    def full(cls, shape, value, dtype=uop.F32, device_id=0):
        shp, nd = _i64(shape)
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_full(device_id, shp, nd, float(value), dtype, C.byref(h)))
        return cls(h)

    # ---- metadata
    @property
    def shape(self):
        nd = lib.mrk_hip_tensor_ndim(self._h)
        out = (C.c_int64 * max(nd, 1))()
        check(lib.mrk_hip_tensor_shape(self._h, out, nd))
        return tuple(out[i] for i in range(nd))

    @property
    def dtype(self):
        return lib.mrk_hip_tensor_dtype(self._h)

    # ---- helpers
    def _new(self, fn, *args):
        h = C.c_void_p()
        check(fn(self._h, *args, C.byref(h)))
        return Tensor(h)

    def _coerce(self, other):
        return other if isinstance(other, Tensor) else Tensor.const(other, self.dtype)

    # ---- movement
    def try_reshape(self, shape):
        shp, nd = _i64(shape)
        return self._new(lib.mrk_hip_tensor_reshape, shp, nd)

    def try_permute(self, perm):
        p, nd = _i64(perm)
        return self._new(lib.mrk_hip_tensor_permute, p, nd)

    def try_transpose(self, a, b):
        return self._new(lib.mrk_hip_tensor_transpose, a, b)

    def try_expand(self, shape):
        shp, nd = _i64(shape)
        return self._new(lib.mrk_hip_tensor_expand, shp, nd)

    def try_shrink(self, ranges):
        b, nd = _i64([r[0] for r in ranges])
        e, _ = _i64([r[1] for r in ranges])
        return self._new(lib.mrk_hip_tensor_shrink, b, e, nd)

    def contiguous(self):
        return self._new(lib.mrk_hip_tensor_contiguous)

    @staticmethod
    def cat(parts, axis):
        arr = (C.c_void_p * len(parts))(*[p._h for p in parts])
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_cat(arr, len(parts), axis, C.byref(h)))
        return Tensor(h)

    # ---- elementwise
    def cast(self, dtype):
        return self._new(lib.mrk_hip_tensor_cast, dtype)

    def unary(self, name):
        return self._new(lib.mrk_hip_tensor_unary, uop.UNARY_OPS[name])

    def binary(self, name, other):
        rhs = self._coerce(other)  # keeps the temporary's handle alive across the call
        return self._new(lib.mrk_hip_tensor_binary, uop.BINARY_OPS[name], rhs._h)

    def try_add(self, o):
        return self.binary("add", o)

    def try_sub(self, o):
        return self.binary("sub", o)

    def try_mul(self, o):
        return self.binary("mul", o)

    def try_div(self, o):
        return self.binary("fdiv", o)

    def maximum(self, o):
        return self.binary("max", o)

    __add__, __sub__, __mul__, __truediv__ = try_add, try_sub, try_mul, try_div

    def where(self, cond, other):
        """cond ? self : other"""
        h = C.c_void_p()
        rhs = self._coerce(other)
        check(lib.mrk_hip_tensor_where(cond._h, self._h, rhs._h, C.byref(h)))
        return Tensor(h)

    def try_exp(self):
        return self.unary("exp")

    def try_exp2(self):
        return self.unary("exp2")

    def try_sqrt(self):
        return self.unary("sqrt")

    def try_rsqrt(self):
        return self.unary("rsqrt")

    def square(self):
        return self.unary("square")

    def sigmoid(self):
        return self._new(lib.mrk_hip_tensor_sigmoid)

    def silu(self):
        return self._new(lib.mrk_hip_tensor_silu)

    def tanh(self):
        return self._new(lib.mrk_hip_tensor_tanh)

    swish = silu

    # ---- reductions
    def reduce(self, op, axes, keepdim=False, promote=True):
        axes = [axes] if isinstance(axes, int) else list(axes)
        a, n = _i64(axes)
        return self._new(lib.mrk_hip_tensor_reduce, uop.REDUCE_OPS[op], a, n, int(keepdim), int(promote))

    def sum(self, axes, keepdim=False):
        return self.reduce("add", axes, keepdim, True)

    def max(self, axes, keepdim=False):
        return self.reduce("max", axes, keepdim, False)

    def mean(self, axes, keepdim=False):
        axes = [axes] if isinstance(axes, int) else list(axes)
        a, n = _i64(axes)
        return self._new(lib.mrk_hip_tensor_mean, a, n, int(keepdim))

    # ---- composite ops
    def matmul(self, other, dtype=None):
        """matmul.rs:82-110 (vector operands included); dtype: accumulate in and return that dtype."""
        if dtype is None:
            return self._new(lib.mrk_hip_tensor_matmul, other._h)
        return self._new(lib.mrk_hip_tensor_matmul_with, other._h, int(dtype))

    dot = matmul

    def gemm(self, b, alpha=1.0, beta=1.0, trans_a=False, trans_b=False, c=None):
        """alpha * op(A) @ op(B) + beta * C (matmul.rs:112-135)."""
        return self._new(lib.mrk_hip_tensor_gemm, b._h, float(alpha), float(beta), int(trans_a), int(trans_b),
                         c._h if c is not None else None)

    def linear(self, weight, bias=None, dtype=None):
        """self @ weight.T + bias, weight [out, in] (matmul.rs:160-190)."""
        return self._new(lib.mrk_hip_tensor_linear, weight._h, bias._h if bias is not None else None,
                         -1 if dtype is None else int(dtype))

    def softmax(self, axis=-1):
        return self._new(lib.mrk_hip_tensor_softmax, axis)

    def log_softmax(self, axis=-1):
        return self._new(lib.mrk_hip_tensor_log_softmax, axis)

    def logsumexp(self, axis=-1):
        return self._new(lib.mrk_hip_tensor_logsumexp, axis)

    def rms_norm(self, axis=-1, eps=1e-5):
        return self._new(lib.mrk_hip_tensor_rms_norm, axis, float(eps))

    def embedding(self, indices):
        """self is the [vocab, dim] weight."""
        return self._new(lib.mrk_hip_tensor_embedding, indices._h)

    def apply_rotary_emb(self, cos, sin, interleaved=False):
        return self._new(lib.mrk_hip_tensor_rotary, cos._h, sin._h, int(interleaved))

    def scaled_dot_product_attention(self, key, value, scale=None, is_causal=False, attn_mask=None, softcap=None):
        """transformer.rs:78-137.  attn_mask: Bool (True = attend) or additive, broadcastable to
        [.., Sq, Sk]; softcap: cap * tanh(scores / cap), applied after the masks.  bf16 operands with a
        Bool or bf16 mask run inside the fused attention kernel."""
        if attn_mask is None and not softcap:
            return self._new(lib.mrk_hip_tensor_sdpa, key._h, value._h, float(scale) if scale else 0.0, int(is_causal))
        return self._new(lib.mrk_hip_tensor_sdpa_ex, key._h, value._h, attn_mask._h if attn_mask is not None else None,
                         float(scale) if scale else 0.0, int(is_causal), float(softcap) if softcap else 0.0)

    # ---- realization / extraction
    def realize(self):
        check(lib.mrk_hip_tensor_realize(self._h))
        return self

    def prepare(self):
        """Tensor::prepare: schedule + compile into an ExecutionPlan without running it."""
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_prepare(self._h, C.byref(h)))
        return ExecutionPlan(_handle=h)

    def kernels(self):
        """Names of the kernels the last realize launched (tensor/src/lib.rs:213)."""
        return last_kernels()

    def to_numpy(self):
        shape = self.shape
        out = np.empty(shape, dtype=_NP_OF[self.dtype])
        check(lib.mrk_hip_tensor_to_bytes(self._h, out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def to_vec(self):
        return self.to_numpy().reshape(-1)

    def as_vec(self):
        """Tensor::as_vec (tensor/src/data.rs:211-236): the flat contents (realizes if needed)."""
        return self.to_vec()

    def buffer(self):
        h = C.c_void_p()
        check(lib.mrk_hip_tensor_buffer(self._h, C.byref(h)))
        n = int(np.prod(self.shape)) * np.dtype(_NP_OF[self.dtype]).itemsize
        return Buffer(n, _handle=h)
