"""Loader of tests/hostshim/libmorok_hostshim.so: the product's host runtime linked against
host-memory stand-ins for the HIP layer (test infrastructure; computes nothing).  The shim
exports the same C ABI as libmorok_hip.so, so the package's ctypes signatures are reused."""
import ctypes as C
import os
import subprocess

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hostshim")
PATH = os.path.join(HERE, "libmorok_hostshim.so")
_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(PATH):
        subprocess.check_call(["make", "-C", HERE], stdout=subprocess.DEVNULL)
    from morok_amd import _ffi

    lib = C.CDLL(PATH, mode=C.RTLD_LOCAL)
    for name, (res, args) in _ffi._SIGS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    for name, res, args in [
        ("mrk_shim_reset", None, []),
        ("mrk_shim_set_memory_limit", None, [C.c_size_t]),
        ("mrk_shim_set_device_count", None, [C.c_int]),
        ("mrk_shim_bytes_in_use", C.c_size_t, []),
        ("mrk_shim_alloc_calls", C.c_size_t, []),
        ("mrk_shim_free_calls", C.c_size_t, []),
        ("mrk_shim_launches", C.c_size_t, []),
        ("mrk_shim_fail_module_load_after", None, [C.c_long]),
        ("mrk_shim_set_events_pending", None, [C.c_int]),
        ("mrk_shim_trace", None, [C.c_int]),
        ("mrk_shim_trace_get", C.c_size_t, [C.c_char_p, C.c_size_t]),
        ("mrk_shim_graph_launches", C.c_size_t, []),
        ("mrk_shim_graphs_alive", C.c_size_t, []),
        ("mrk_shim_syncs", C.c_size_t, []),
        ("mrk_shim_last_kernel", C.c_char_p, []),
        ("mrk_shim_last_dims", None, [C.POINTER(C.c_uint * 3), C.POINTER(C.c_uint * 3)]),
    ]:
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_dims(lib):
    g, b = (C.c_uint * 3)(), (C.c_uint * 3)()
    lib.mrk_shim_last_dims(C.byref(g), C.byref(b))
    return tuple(g), tuple(b)


def trace(lib):
    """The stream operations recorded since mrk_shim_trace(1), as a list of strings."""
    n = lib.mrk_shim_trace_get(None, 0)
    buf = C.create_string_buffer(n + 1)
    lib.mrk_shim_trace_get(buf, n + 1)
    return buf.value.decode().split()
