"""Thin Python mirrors of the boundary objects, forwarding to the C ABI.

Names follow the reference (device/src/device.rs, device/src/buffer.rs): Device, Buffer
(lazy allocation, views, copyin/copyout/copy_from), ProgramSpec, CompiledSpec, Program
(`execute(buffers, vals, global_size, local_size)`).
"""
import ctypes as C

import numpy as np

from . import _ffi
from ._ffi import MorokHipError, check, lib


def parse_device(spec: str) -> int:
    """DeviceSpecExt::parse (device/src/registry.rs:26-81) for the HIP arm."""
    out = C.c_int(0)
    check(lib.mrk_hip_device_parse(spec.encode(), C.byref(out)))
    return out.value


def device_count() -> int:
    out = C.c_int(0)
    check(lib.mrk_hip_device_count(C.byref(out)))
    return out.value


class Buffer:
    """device::Buffer (device/src/buffer.rs:97-574)."""

    def __init__(self, size, device_id=0, zero_init=False, cpu_accessible=False, _handle=None):
        if _handle is not None:
            self._h = _handle
        else:
            h = C.c_void_p()
            check(lib.mrk_hip_buffer_new(device_id, size, int(zero_init), int(cpu_accessible), C.byref(h)))
            self._h = h
        self.device_id = device_id

    @classmethod
    def from_numpy(cls, arr, device_id=0):
        arr = np.ascontiguousarray(arr)
        b = cls(arr.nbytes, device_id)
        b.copyin(arr)
        return b

    def ensure_allocated(self):
        check(lib.mrk_hip_buffer_ensure_allocated(self._h))
        return self

    def is_allocated(self):
        return bool(lib.mrk_hip_buffer_is_allocated(self._h))

    def view(self, offset, size):
        h = C.c_void_p()
        check(lib.mrk_hip_buffer_view(self._h, offset, size, C.byref(h)))
        return Buffer(size, self.device_id, _handle=h)

    def copyin(self, data):
        if isinstance(data, np.ndarray):
            data = np.ascontiguousarray(data)
            check(lib.mrk_hip_buffer_copyin(self._h, data.ctypes.data_as(C.c_void_p), data.nbytes))
        else:
            raw = bytes(data)
            check(lib.mrk_hip_buffer_copyin(self._h, C.cast(C.c_char_p(raw), C.c_void_p), len(raw)))
        return self

    def copyout(self, dtype=np.uint8, shape=None, nbytes=None):
        n = self.size if nbytes is None else nbytes
        out = np.empty(n, dtype=np.uint8)
        check(lib.mrk_hip_buffer_copyout(self._h, out.ctypes.data_as(C.c_void_p), n))
        out = out.view(dtype)
        return out.reshape(shape) if shape is not None else out

    def copy_from(self, src):
        check(lib.mrk_hip_buffer_copy_from(self._h, src._h))
        return self

    @property
    def ptr(self):
        """as_raw_ptr: device address (allocates on first use like the execution plan does)."""
        self.ensure_allocated()
        p = C.c_void_p()
        check(lib.mrk_hip_buffer_raw_ptr(self._h, C.byref(p)))
        return p.value

    def raw_ptr_unallocated_ok(self):
        p = C.c_void_p()
        check(lib.mrk_hip_buffer_raw_ptr(self._h, C.byref(p)))
        return p.value

    @property
    def id(self):
        return lib.mrk_hip_buffer_id(self._h)

    @property
    def size(self):
        return lib.mrk_hip_buffer_size(self._h)

    def synchronize(self):
        check(lib.mrk_hip_buffer_synchronize(self._h))

    def release(self):
        if self._h is not None and self._h.value:
            lib.mrk_hip_buffer_release(self._h)
            self._h = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def _size3(v):
    if v is None:
        return None
    arr = (C.c_size_t * 3)(*[int(x) for x in v])
    return arr


class ProgramSpec:
    """device::ProgramSpec (device/src/device.rs:327-367)."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def from_source(cls, name, src, buf_count, var_names=(), var_is_i64=None, global_size=None, local_size=None):
        n = len(var_names)
        names = (C.c_char_p * max(n, 1))(*[v.encode() for v in var_names])
        flags = (C.c_uint8 * max(n, 1))(*[int(bool(x)) for x in (var_is_i64 or [0] * n)])
        h = C.c_void_p()
        check(
            lib.mrk_hip_program_spec_from_source(
                name.encode(), src.encode(), buf_count, names, flags, n, _size3(global_size), _size3(local_size),
                C.byref(h)
            )
        )
        return cls(h)

    @property
    def name(self):
        return lib.mrk_hip_program_spec_name(self._h).decode()

    @property
    def src(self):
        return lib.mrk_hip_program_spec_src(self._h).decode()

    @property
    def buf_count(self):
        return lib.mrk_hip_program_spec_buf_count(self._h)

    @property
    def var_names(self):
        return [lib.mrk_hip_program_spec_var_name(self._h, i).decode()
                for i in range(lib.mrk_hip_program_spec_var_count(self._h))]

    def sizes(self):
        g = (C.c_size_t * 3)()
        l = (C.c_size_t * 3)()
        if not lib.mrk_hip_program_spec_sizes(self._h, g, l):
            return None, None
        return list(g), list(l)

    @property
    def global_size(self):
        return self.sizes()[0]

    @property
    def local_size(self):
        return self.sizes()[1]

    def _slots(self, which):
        buf = (C.c_size_t * 64)()
        n = lib.mrk_hip_program_spec_slots(self._h, which, buf, 64)
        return list(buf[: min(n, 64)])

    @property
    def globals(self):
        return self._slots(0)

    @property
    def outs(self):
        return self._slots(1)

    @property
    def ins(self):
        return self._slots(2)

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_program_spec_release(self._h)
                self._h = None
        except Exception:
            pass


class CompiledSpec:
    """device::CompiledSpec (device/src/device.rs:72-100)."""

    def __init__(self, handle):
        self._h = handle

    @property
    def name(self):
        return lib.mrk_hip_compiled_spec_name(self._h).decode()

    @property
    def bytes(self):
        p = C.POINTER(C.c_uint8)()
        n = lib.mrk_hip_compiled_spec_bytes(self._h, C.byref(p))
        return C.string_at(p, n)

    @property
    def src(self):
        return None if not lib.mrk_hip_compiled_spec_has_src(self._h) else ""

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_compiled_spec_release(self._h)
                self._h = None
        except Exception:
            pass


def compile_spec(spec: ProgramSpec) -> CompiledSpec:
    """Compiler::compile (device/src/device.rs:170)."""
    h = C.c_void_p()
    check(lib.mrk_hip_compile(spec._h, C.byref(h)))
    return CompiledSpec(h)


def cache_key() -> str:
    return lib.mrk_hip_cache_key().decode()


class Program:
    """Box<dyn Program> (device/src/device.rs:34-60)."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def create(cls, compiled: CompiledSpec, device_id=0):
        """RuntimeFactory (device/src/device.rs:234)."""
        h = C.c_void_p()
        check(lib.mrk_hip_program_create(device_id, compiled._h, C.byref(h)))
        return cls(h)

    @classmethod
    def builtin(cls, kind, params, device_id=0):
        arr = (C.c_int64 * max(len(params), 1))(*[int(p) for p in params])
        h = C.c_void_p()
        check(lib.mrk_hip_program_builtin(device_id, kind.encode(), arr, len(params), C.byref(h)))
        return cls(h)

    def execute(self, buffers, vals=(), global_size=None, local_size=None):
        ptrs = [b.ptr if isinstance(b, Buffer) else int(b) for b in buffers]
        parr = (C.c_void_p * max(len(ptrs), 1))(*ptrs)
        varr = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
        check(
            lib.mrk_hip_program_execute(
                self._h, parr, len(ptrs), varr, len(vals), _size3(global_size), _size3(local_size)
            )
        )

    @property
    def name(self):
        return lib.mrk_hip_program_name(self._h).decode()

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_program_destroy(self._h)
                self._h = None
        except Exception:
            pass


class Device:
    """The HIP device bundle (device/src/device.rs:255-313), looked up through the factory
    registry under the base type "HIP" (runtime/src/device_registry.rs:99-127)."""

    def __init__(self, spec="HIP"):
        self.device_id = parse_device(spec) if isinstance(spec, str) else int(spec)
        check(lib.mrk_hip_device_create(self.device_id))

    base_device_key = staticmethod(lambda: lib.mrk_hip_name().decode())

    def synchronize(self):
        check(lib.mrk_hip_sync(self.device_id))

    def alloc(self, size, zero_init=False, cpu_accessible=False):
        p = C.c_void_p()
        check(lib.mrk_hip_alloc(self.device_id, size, int(zero_init), int(cpu_accessible), C.byref(p)))
        return p.value

    def free(self, ptr, size, cpu_accessible=False):
        check(lib.mrk_hip_free(self.device_id, ptr, size, int(cpu_accessible)))

    def lru_cache_count(self, size, cpu_accessible=False):
        n = C.c_size_t()
        check(lib.mrk_hip_lru_cache_count(self.device_id, size, int(cpu_accessible), C.byref(n)))
        return n.value

    def lru_total_cached(self):
        n = C.c_size_t()
        check(lib.mrk_hip_lru_total_cached(self.device_id, C.byref(n)))
        return n.value

    def lru_clear(self):
        check(lib.mrk_hip_lru_clear(self.device_id))

    def buffer(self, size, **kw):
        return Buffer(size, self.device_id, **kw)


class Event:
    def __init__(self, device_id=0):
        h = C.c_void_p()
        check(lib.mrk_hip_event_create(device_id, C.byref(h)))
        self._h = h

    def record(self):
        check(lib.mrk_hip_event_record(self._h))
        return self

    def synchronize(self):
        check(lib.mrk_hip_event_synchronize(self._h))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        check(lib.mrk_hip_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_event_destroy(self._h)
                self._h = None
        except Exception:
            pass


def time_launches(fn, iters, warmup=3, device_id=0):
    """Average milliseconds per call of `fn` over `iters` launches, measured with HIP
    events recorded on the device's own stream."""
    for _ in range(warmup):
        fn()
    e0, e1 = Event(device_id), Event(device_id)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_ms(e1) / iters


def time_each_launch(fn, iters, warmup=3, device_id=0):
    """Per-launch milliseconds (one event pair per call): returns (median, minimum)."""
    for _ in range(warmup):
        fn()
    events = [Event(device_id) for _ in range(iters + 1)]
    events[0].record()
    for i in range(iters):
        fn()
        events[i + 1].record()
    events[-1].synchronize()
    ms = sorted(events[i].elapsed_ms(events[i + 1]) for i in range(iters))
    return ms[len(ms) // 2], ms[0]


class Kernel:
    """Arc<CachedKernel> (runtime/src/kernel_cache.rs:27-44), obtained through the global
    kernel cache."""

    def __init__(self, handle, was_cached=False):
        self._h = handle
        self.was_cached = was_cached

    @classmethod
    def get_or_compile(cls, kernel, name=None, device_id=0):
        """get_or_compile_kernel (kernel_cache.rs:87-118) over render -> compile -> runtime."""
        data = kernel.serialize() if hasattr(kernel, "serialize") else bytes(kernel)
        h = C.c_void_p()
        cached = C.c_int(0)
        check(lib.mrk_hip_kernel_get_or_compile(device_id, data, len(data), name.encode() if name else None,
                                                C.byref(h), C.byref(cached)))
        return cls(h, bool(cached.value))

    @classmethod
    def builtin(cls, kind, params, device_id=0):
        arr = (C.c_int64 * max(len(params), 1))(*[int(p) for p in params])
        h = C.c_void_p()
        check(lib.mrk_hip_kernel_builtin(device_id, kind.encode(), arr, len(params), C.byref(h)))
        return cls(h)

    @property
    def entry_point(self):
        return lib.mrk_hip_kernel_entry_point(self._h).decode()

    @property
    def code(self):
        return lib.mrk_hip_kernel_code(self._h).decode()

    @property
    def var_names(self):
        return [lib.mrk_hip_kernel_var_name(self._h, i).decode() for i in range(lib.mrk_hip_kernel_var_count(self._h))]

    def same_as(self, other):
        return bool(lib.mrk_hip_kernel_same(self._h, other._h))

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_kernel_release(self._h)
                self._h = None
        except Exception:
            pass


def kernel_cache_size():
    return lib.mrk_hip_kernel_cache_size()


def kernel_cache_clear():
    lib.mrk_hip_kernel_cache_clear()


class ExecutionPlan:
    """ExecutionPlan + builder (runtime/src/execution_plan.rs:84-250,330-411)."""

    def __init__(self, device_id=0, _handle=None):
        if _handle is not None:
            self._h = _handle
        else:
            h = C.c_void_p()
            check(lib.mrk_hip_plan_create(device_id, C.byref(h)))
            self._h = h
        self._buffers = []

    def add_buffer(self, buf):
        idx = C.c_size_t()
        check(lib.mrk_hip_plan_add_buffer(self._h, buf._h, C.byref(idx)))
        self._buffers.append(buf)
        return idx.value

    def add_kernel(self, kernel, buffer_indices, vals=()):
        bi = (C.c_size_t * max(len(buffer_indices), 1))(*buffer_indices)
        va = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
        check(lib.mrk_hip_plan_add_kernel(self._h, kernel._h, bi, len(buffer_indices), va, len(vals)))

    def build(self):
        check(lib.mrk_hip_plan_build(self._h))
        return self

    def execute(self):
        check(lib.mrk_hip_plan_execute(self._h))

    def execute_graph(self):
        """The same launches replayed as one HIP graph (recorded on the first call)."""
        check(lib.mrk_hip_plan_execute_graph(self._h))

    def execute_profiled(self):
        n = lib.mrk_hip_plan_kernel_count(self._h)
        ms = (C.c_double * max(n, 1))()
        cnt = C.c_size_t()
        check(lib.mrk_hip_plan_execute_profiled(self._h, ms, n, C.byref(cnt)))
        return [(self.kernel_name(i), ms[i]) for i in range(cnt.value)]

    def execute_with_vars(self, var_vals):
        names = (C.c_char_p * max(len(var_vals), 1))(*[k.encode() for k in var_vals])
        vals = (C.c_int64 * max(len(var_vals), 1))(*[int(v) for v in var_vals.values()])
        check(lib.mrk_hip_plan_execute_with_vars(self._h, names, vals, len(var_vals)))

    @property
    def kernel_count(self):
        return lib.mrk_hip_plan_kernel_count(self._h)

    def kernel_name(self, i):
        return lib.mrk_hip_plan_kernel_name(self._h, i).decode()

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_plan_release(self._h)
                self._h = None
        except Exception:
            pass


def benchmark_kernel(program, buffers, vals=(), global_size=None, local_size=None, warmup=1, runs=3, device_id=0):
    """benchmark_kernel (runtime/src/benchmark.rs:64-91): (min_ms, mean_ms) with the reference's
    default protocol of 1 warm-up and 3 timed runs."""
    ptrs = [b.ptr if isinstance(b, Buffer) else int(b) for b in buffers]
    parr = (C.c_void_p * max(len(ptrs), 1))(*ptrs)
    varr = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
    mn, mean = C.c_double(), C.c_double()
    check(lib.mrk_hip_benchmark_kernel(device_id, program._h, parr, len(ptrs), varr, len(vals), _size3(global_size),
                                       _size3(local_size), warmup, runs, C.byref(mn), C.byref(mean)))
    return mn.value, mean.value


def benchmark_kernel_with_cutoff(program, buffers, cutoff_ms, vals=(), global_size=None, local_size=None, warmup=1, runs=3,
                                 device_id=0):
    """benchmark_kernel_with_cutoff (runtime/src/benchmark.rs:100-137): None when the first timed
    run took more than three times `cutoff_ms` (the candidate is given up), else (min_ms, mean_ms)."""
    ptrs = [b.ptr if isinstance(b, Buffer) else int(b) for b in buffers]
    parr = (C.c_void_p * max(len(ptrs), 1))(*ptrs)
    varr = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
    mn, mean, skipped = C.c_double(), C.c_double(), C.c_int()
    check(lib.mrk_hip_benchmark_kernel_with_cutoff(device_id, program._h, parr, len(ptrs), varr, len(vals), _size3(global_size),
                                                   _size3(local_size), warmup, runs, float(cutoff_ms), C.byref(mn),
                                                   C.byref(mean), C.byref(skipped)))
    return None if skipped.value else (mn.value, mean.value)


class TimelineSignal:
    """TimelineSignal over HIP events (device/src/sync.rs:44-71,192-310)."""

    def __init__(self, device_id=0):
        h = C.c_void_p()
        check(lib.mrk_hip_signal_create(device_id, C.byref(h)))
        self._h = h

    def set(self, value):
        check(lib.mrk_hip_signal_set(self._h, value))

    @property
    def value(self):
        return lib.mrk_hip_signal_value(self._h)

    def wait(self, value, timeout_ms):
        check(lib.mrk_hip_signal_wait(self._h, value, timeout_ms))

    def is_reached(self, value):
        return self.value >= value

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_signal_destroy(self._h)
                self._h = None
        except Exception:
            pass


class HardwareQueue:
    """HardwareQueue (device/src/queue.rs:76-141): batches commands for its own HIP stream;
    submit() hands them over without waiting.  The library keeps the buffers and kernels of a
    submitted batch referenced until it has run, so callers may drop theirs after submit().
    Every method returns self for chaining."""

    def __init__(self, device_id=0, copy_queue=False):
        h = C.c_void_p()
        check(lib.mrk_hip_queue_create(device_id, int(copy_queue), C.byref(h)))
        self._h = h

    def wait(self, signal, value):
        check(lib.mrk_hip_queue_wait(self._h, signal._h, value))
        return self

    def signal(self, signal, value):
        check(lib.mrk_hip_queue_signal(self._h, signal._h, value))
        return self

    def exec(self, kernel, buffers, vals=(), global_size=None, local_size=None):
        bufs = (C.c_void_p * max(len(buffers), 1))(*[b._h for b in buffers])
        va = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
        g = _size3(global_size) if global_size is not None else None
        l = _size3(local_size) if local_size is not None else None
        check(lib.mrk_hip_queue_exec(self._h, kernel._h, bufs, len(buffers), va, len(vals), g, l))
        return self

    def copy(self, dst, src):
        check(lib.mrk_hip_queue_copy(self._h, dst._h, src._h))
        return self

    def memory_barrier(self):
        check(lib.mrk_hip_queue_memory_barrier(self._h))
        return self

    def submit(self, wait_timeout_ms=10000):
        check(lib.mrk_hip_queue_submit(self._h, wait_timeout_ms))
        return self

    def synchronize(self):
        check(lib.mrk_hip_queue_synchronize(self._h))
        return self

    @property
    def pending(self):
        return lib.mrk_hip_queue_pending(self._h)

    def __del__(self):
        try:
            if self._h:
                lib.mrk_hip_queue_destroy(self._h)
                self._h = None
        except Exception:
            pass
