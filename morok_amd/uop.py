"""Builder and serializer for linearized UOp kernels - the input of Renderer::render.

A kernel is the flat, already-ordered node list that morok's linearizer hands to a
renderer (schedule/src/linearize/mod.rs:172-177,308-310; vocabulary ir/src/op.rs:33-305).
This module only *describes* kernels (ids, ops, dtypes, sources, arguments) and packs them
into the wire format of morok_amd/csrc/uop.h; rendering, compiling and running happen in
libmorok_hip.so.
"""
import ctypes as C
import struct

from ._ffi import check, lib
from .device import ProgramSpec

# ---- enums (must match morok_amd/csrc/uop.h)
(PARAM, DEFINE_VAR, DEFINE_LOCAL, DEFINE_REG, CONST, SPECIAL, RANGE, END, INDEX, LOAD, STORE, UNARY, BINARY, WHERE,
 MULACC, CAST, BITCAST, GEP, VECTORIZE, WMMA, IF, ENDIF, BARRIER, AFTER, NOOP, SINK, REDUCE, WAVE_REDUCE, LOAD_TR, ASYNC_COPY,
 WAIT_ASYNC) = range(31)

(BOOL, I8, U8, I16, U16, I32, U32, I64, U64, F16, BF16, F32, F64, VOID, INDEX_T, FP8E4M3, FP8E5M2) = range(17)
GLOBAL, LOCAL, REG = 0, 1, 2
(AX_GLOBAL, AX_WARP, AX_LOCAL, AX_LOOP, AX_GROUP_REDUCE, AX_REDUCE, AX_UPCAST, AX_UNROLL, AX_THREAD, AX_OUTER) = range(10)

UNARY_OPS = {n: i for i, n in enumerate(
    ["neg", "abs", "sqrt", "rsqrt", "reciprocal", "exp", "exp2", "log", "log2", "sin", "cos", "tan", "floor", "ceil",
     "trunc", "round", "erf", "sign", "square", "not"])}
BINARY_OPS = {n: i for i, n in enumerate(
    ["add", "sub", "mul", "fdiv", "mod", "max", "pow", "and", "or", "xor", "shl", "shr", "idiv", "lt", "le", "gt", "ge",
     "eq", "ne", "threefry"])}
REDUCE_OPS = {"add": 0, "mul": 1, "max": 2, "min": 3}
_CMP = {"lt", "le", "gt", "ge", "eq", "ne"}
_FLOATS = {F16, BF16, F32, F64}


class DT:
    """A dtype: scalar tag, vector width, optional pointer (address space, element count)."""

    __slots__ = ("scalar", "vcount", "ptr", "space", "size")

    def __init__(self, scalar, vcount=1, ptr=False, space=GLOBAL, size=-1):
        self.scalar, self.vcount, self.ptr, self.space, self.size = scalar, vcount, ptr, space, size

    def vec(self, n):
        return DT(self.scalar, n)

    def scalar_of(self):
        return DT(self.scalar)

    def ptr_to(self, size=-1, space=GLOBAL):
        return DT(self.scalar, self.vcount, True, space, size)

    def base(self):
        return DT(self.scalar, self.vcount)

    @property
    def is_float(self):
        return self.scalar in _FLOATS


f32, f16, bf16, f64 = DT(F32), DT(F16), DT(BF16), DT(F64)
fp8e4m3, fp8e5m2 = DT(FP8E4M3), DT(FP8E5M2)   # one byte each; tensor-core operands only
i32, i64, u32, u8, i8, boolean, index = DT(I32), DT(I64), DT(U32), DT(U8), DT(I8), DT(BOOL), DT(INDEX_T)


class Kernel:
    """Append-only linearized kernel.  Every method returns the id of the node it adds."""

    def __init__(self):
        self.nodes = []
        self.dtypes = {}

    def _add(self, op, dt, src=(), arg_i=0, arg_f=0.0, sub=0, s="", extra=()):
        nid = len(self.nodes) + 1
        self.nodes.append((nid, op, dt, tuple(src), int(arg_i), float(arg_f), int(sub), s, tuple(int(e) for e in extra)))
        self.dtypes[nid] = dt
        return nid

    # ---- definitions
    def param(self, slot, dt, size=-1):
        return self._add(PARAM, dt.ptr_to(size), arg_i=slot)

    def define_var(self, name, dt=i32, lo=0, hi=0):
        return self._add(DEFINE_VAR, dt, s=name, extra=(lo, hi))

    def define_local(self, lid, dt, size):
        return self._add(DEFINE_LOCAL, dt.ptr_to(size, LOCAL), arg_i=lid)

    def define_reg(self, rid, dt, size):
        return self._add(DEFINE_REG, dt.ptr_to(size, REG), arg_i=rid)

    def const(self, value, dt=i32):
        if dt.is_float:
            return self._add(CONST, dt, arg_f=value)
        return self._add(CONST, dt, arg_i=int(value))

    def special(self, name, extent, dt=i32):
        return self._add(SPECIAL, dt, src=(self.const(extent, dt),), s=name)

    # ---- control flow
    def range(self, end, axis_id, axis_type=AX_LOOP, dt=i32):
        end_id = end.id if isinstance(end, _Ref) else self.const(end, dt)
        return self._add(RANGE, dt, src=(end_id,), arg_i=axis_id, sub=axis_type)

    def end(self, *ranges):
        return self._add(END, DT(VOID), src=ranges)

    def if_(self, cond):
        return self._add(IF, DT(VOID), src=(cond,))

    def endif(self):
        return self._add(ENDIF, DT(VOID))

    def barrier(self, src=None):
        return self._add(BARRIER, DT(VOID), src=(src,) if src else ())

    # ---- memory
    def index(self, buf, idx, gate=None, strides=None):
        idxs = idx if isinstance(idx, (list, tuple)) else [idx]
        src = [buf] + list(idxs) + ([gate] if gate is not None else [])
        return self._add(INDEX, self.dtypes[buf], src=src, sub=1 if gate is not None else 0, extra=strides or ())

    def load(self, idx, alt=None, dt=None):
        dt = dt or self.dtypes[idx].base()
        return self._add(LOAD, dt, src=(idx,) + ((alt,) if alt is not None else ()))

    def store(self, idx, value):
        return self._add(STORE, DT(VOID), src=(idx, value))

    # ---- ALU
    def unary(self, op, x):
        return self._add(UNARY, self.dtypes[x], src=(x,), sub=UNARY_OPS[op])

    def binary(self, op, a, b):
        dt = boolean.vec(self.dtypes[a].vcount) if op in _CMP and self.dtypes[a].vcount > 1 else (
            boolean if op in _CMP else self.dtypes[a])
        return self._add(BINARY, dt, src=(a, b), sub=BINARY_OPS[op])

    def where(self, c, t, f):
        return self._add(WHERE, self.dtypes[t], src=(c, t, f))

    def mulacc(self, a, b, c):
        return self._add(MULACC, self.dtypes[c], src=(a, b, c))

    def cast(self, x, dt):
        return self._add(CAST, dt, src=(x,))

    def bitcast(self, x, dt):
        return self._add(BITCAST, dt, src=(x,))

    def gep(self, v, *indices):
        dt = self.dtypes[v].scalar_of() if len(indices) == 1 else self.dtypes[v].vec(len(indices))
        return self._add(GEP, dt, src=(v,), extra=indices)

    def vectorize(self, *elems):
        return self._add(VECTORIZE, self.dtypes[elems[0]].vec(len(elems)), src=elems)

    def wmma(self, a, b, c, name):
        return self._add(WMMA, self.dtypes[c], src=(a, b, c), s=name)

    def reduce(self, op, value, *ranges):
        return self._add(REDUCE, self.dtypes[value], src=(value,) + ranges, sub=REDUCE_OPS[op])

    def wave_reduce(self, op, value):
        return self._add(WAVE_REDUCE, self.dtypes[value], src=(value,), sub=REDUCE_OPS[op])

    def load_tr(self, local_index):
        """Transposing load of four 16-bit elements from local memory (extension op LOAD_TR)."""
        return self._add(LOAD_TR, DT(self.dtypes[local_index].scalar, 4), src=(local_index,))

    def async_copy(self, global_index, local_index):
        """Direct global -> local copy of 16 bytes per lane; the local index must be the same for the
        64 lanes of a wave, lane i lands 16 * i bytes behind it (extension op ASYNC_COPY)."""
        return self._add(ASYNC_COPY, DT(VOID), src=(global_index, local_index))

    def wait_async(self, n):
        """Waits until at most n of the wave's async copies are in flight (extension op WAIT_ASYNC)."""
        return self._add(WAIT_ASYNC, DT(VOID), arg_i=n)

    def after(self, x, *deps):
        return self._add(AFTER, self.dtypes[x], src=(x,) + deps)

    def sink(self, *srcs):
        return self._add(SINK, DT(VOID), src=srcs)

    # convenience
    def add(self, a, b):
        return self.binary("add", a, b)

    def mul(self, a, b):
        return self.binary("mul", a, b)

    # ---- wire format
    def serialize(self):
        out = [struct.pack("<III", 0x4C4B524D, 1, len(self.nodes))]
        for nid, op, dt, src, arg_i, arg_f, sub, s, extra in self.nodes:
            flags = (1 if dt.ptr else 0) | (dt.space << 1)
            out.append(struct.pack("<IHBBHqH", nid, op, dt.scalar, flags, dt.vcount, dt.size, len(src)))
            out.append(struct.pack("<%dI" % len(src), *src))
            sb = s.encode()
            out.append(struct.pack("<qdHH", arg_i, arg_f, sub, len(sb)))
            out.append(sb)
            out.append(struct.pack("<H%dq" % len(extra), len(extra), *extra))
        return b"".join(out)


class _Ref:
    """Marks an existing node id where a method otherwise takes a Python constant."""

    def __init__(self, nid):
        self.id = nid


def ref(nid):
    return _Ref(nid)


def render(kernel, name=None, device_id=0):
    """Renderer::render (device/src/device.rs:186-222) through the C ABI."""
    data = kernel.serialize() if isinstance(kernel, Kernel) else bytes(kernel)
    h = C.c_void_p()
    check(lib.mrk_hip_render(device_id, data, len(data), name.encode() if name else None, C.byref(h)))
    return ProgramSpec(h)
