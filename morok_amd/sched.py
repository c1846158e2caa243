"""Bindings of the scheduling helpers (capabilities, tensor cores, GPU dims, matmul kernels)."""
import ctypes as C

from ._ffi import check, lib
from . import uop as U


def caps():
    """Renderer::amd_cdna4() (schedule/src/optimizer/renderer.rs:290-303) as a dict."""
    out = {}
    for item in lib.mrk_hip_sched_caps().decode().split(";"):
        k, v = item.split("=", 1)
        out[k] = v
    out["global_max"] = [int(x) for x in out["global_max"].split(",")]
    out["tensor_cores"] = out["tensor_cores"].split(",")
    for k in ("has_local", "has_shared", "has_threads", "shared_max", "local_max", "upcast_max"):
        out[k] = int(out[k])
    return out


def tc_select(in0, in1, acc):
    return lib.mrk_hip_sched_tc_select(in0, in1, acc)


def tc_info(i):
    dims, ept, thr = (C.c_int * 3)(), (C.c_int * 3)(), C.c_int()
    check(lib.mrk_hip_sched_tc_info(i, dims, C.byref(thr), ept))
    return list(dims), thr.value, list(ept)


def tc_element(i, operand, lane, elem):
    a, b = C.c_int(), C.c_int()
    check(lib.mrk_hip_sched_tc_operand_element(i, operand, lane, elem, C.byref(a), C.byref(b)))
    return a.value, b.value


def _arr(v):
    return (C.c_size_t * max(len(v), 1))(*v)


def _dims_call(fn, dims, max_sizes):
    out = (C.c_size_t * 16)()
    n = C.c_size_t()
    rc = fn(_arr(dims), len(dims), _arr(max_sizes), len(max_sizes), out, 16, C.byref(n))
    return rc, list(out[: n.value])


def find_smallest_divisor(n):
    return lib.mrk_hip_sched_find_smallest_divisor(n)


def group_dims(dims, max_sizes):
    rc, out = _dims_call(lib.mrk_hip_sched_group_dims, dims, max_sizes)
    return out if rc == 1 else None


def split_dims(dims, max_sizes):
    return _dims_call(lib.mrk_hip_sched_split_dims, dims, max_sizes)[1]


def limit_dims(dims, max_sizes):
    return _dims_call(lib.mrk_hip_sched_limit_dims, dims, max_sizes)[1]


def get_contraction(original, limited):
    g = (C.c_size_t * max(len(original), 1))()
    if not lib.mrk_hip_sched_get_contraction(_arr(original), len(original), _arr(limited), len(limited), g):
        return None
    groups = [[] for _ in limited]
    for d in range(len(original)):
        groups[g[d]].append(d)
    return groups


def grouped_dims(dims, max_sizes, reverse, raw=None):
    launch = (C.c_size_t * 16)()
    n = C.c_size_t()
    idx = (C.c_size_t * max(len(dims), 1))()
    check(lib.mrk_hip_sched_grouped_dims(_arr(dims), len(dims), _arr(max_sizes) if max_sizes else None,
                                         len(max_sizes) if max_sizes else 0, int(reverse), launch, 16, C.byref(n),
                                         _arr(raw) if raw is not None else None, idx if raw is not None else None))
    return list(launch[: n.value]), (list(idx[: len(dims)]) if raw is not None else None)


def _take(fn, *args):
    p = C.POINTER(C.c_uint8)()
    n = C.c_size_t()
    check(fn(*args, C.byref(p), C.byref(n)))
    data = C.string_at(p, n.value)
    lib.mrk_hip_sched_free(p)
    return data


def build_matmul_f32(m, n, k):
    return _take(lib.mrk_hip_sched_build_matmul_f32, m, n, k)


def build_wmma_matmul(tc_index, m, n, k, out_scalar=U.BF16):
    return _take(lib.mrk_hip_sched_build_wmma_matmul, tc_index, m, n, k, out_scalar)


def build_wmma_matmul_lds(tc_index, m, n, k, out_scalar):
    """The tensor-core matmul with both operands staged through local memory by a workgroup of
    2 x 2 waves (128 x 128 output tile); serialized linear kernel."""
    return _take(lib.mrk_hip_sched_build_wmma_matmul_lds, tc_index, m, n, k, out_scalar)


def build_wmma_matmul_lds_opts(tc_index, m, n, k, out_scalar, opts):
    """The same with explicit (waves_m, waves_n, tiles_m per wave, tiles_n per wave, K steps per
    barrier pair; 0 = by K[, stages: 0 = through registers, 2 = direct global -> local copies, 3 = the
    same with a third stage of the second operand (at most four waves, more than two K steps)])."""
    opts = list(opts) + [0] * (6 - len(opts))
    arr = (C.c_int * 6)(*opts)
    return _take(lib.mrk_hip_sched_build_wmma_matmul_lds_opts, tc_index, m, n, k, out_scalar, arr)


def build_matmul_f32_opts(m, n, k, opts):
    """f32 matmul kernel with explicit (LOCAL x, LOCAL y, UPCAST n, UPCAST m, UNROLL k[, GROUP depth:
    0 or the K depth of the tiles staged through local memory])."""
    arr = (C.c_int * 6)(*(list(opts) + [0] * (6 - len(opts))))
    return _take(lib.mrk_hip_sched_build_matmul_f32_opts, m, n, k, arr)


def compile_and_time(kernel_bytes, buffers, vals=(), name=None, warmup=1, runs=3, device_id=0):
    """Beam-search timing hook: compile (not timed), then the minimum of `runs` event-timed
    launches in milliseconds (tensor/src/realize.rs:1190-1242)."""
    ms = C.c_double()
    bufs = (C.c_void_p * max(len(buffers), 1))(*[b._h for b in buffers])
    va = (C.c_int64 * max(len(vals), 1))(*[int(v) for v in vals])
    check(lib.mrk_hip_compile_and_time(device_id, kernel_bytes, len(kernel_bytes), name.encode() if name else None,
                                       bufs, len(buffers), va, len(vals), warmup, runs, C.byref(ms)))
    return ms.value


def beam_cache_get(ast_hash, width, device):
    buf = C.create_string_buffer(4096)
    n = C.c_size_t()
    check(lib.mrk_hip_beam_cache_get(ast_hash, width, device.encode(), buf, 4096, C.byref(n)))
    return buf.raw[: n.value] if n.value else None


def beam_cache_put(ast_hash, width, device, value):
    check(lib.mrk_hip_beam_cache_put(ast_hash, width, device.encode(), value, len(value)))


def beam_search_matmul_f32(m, n, k, width=2, device_id=0):
    """Returns (opts, best_ms, from_cache, candidates_timed)."""
    opts = (C.c_int * 6)()
    ms = C.c_double()
    cached, timed = C.c_int(), C.c_int()
    check(lib.mrk_hip_beam_search_matmul_f32(device_id, m, n, k, width, opts, C.byref(ms), C.byref(cached), C.byref(timed)))
    return list(opts), ms.value, bool(cached.value), timed.value


def beam_search_wmma_matmul(tc_index, m, n, k, width=2, device_id=0):
    """Beam search over the LDS-staged tensor-core matmul; returns (opts, best_ms, from_cache,
    candidates_timed) with opts as build_wmma_matmul_lds_opts takes them."""
    opts = (C.c_int * 6)()
    ms = C.c_double()
    cached, timed = C.c_int(), C.c_int()
    check(lib.mrk_hip_beam_search_wmma_matmul(device_id, tc_index, m, n, k, width, opts, C.byref(ms), C.byref(cached),
                                              C.byref(timed)))
    return list(opts), ms.value, bool(cached.value), timed.value
