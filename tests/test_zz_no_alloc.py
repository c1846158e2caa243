"""mrk_hip_gemm_bf16_noalloc: the bf16 product for callers that cannot allocate.  Its split-K
partials live in a fixed device array inside the library; everything else is the code of
mrk_hip_gemm_bf16, so the two must agree bit for bit.  Collected last on purpose: the calls
share one array per device and the array keeps the previous call's contents, so the checks run
two calls in a row, the second on a smaller input, both after the rest of the suite and in a
fresh process."""
import numpy as np
import pytest

import morok_amd
from morok_amd import MorokHipError, ops, synth
from morok_amd._ffi import lib

pytestmark = pytest.mark.gpu


def _pair(dev, M, N, K, seed):
    a = synth.normal_bf16((M, K), seed, 0)
    b = synth.normal_bf16((K, N), seed, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)
    want, got = dev.buffer(M * N * 2), dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, want, M, N, K, dev.device_id)
    ops.gemm_bf16_noalloc(ba, bb, got, M, N, K, dev.device_id)
    return got.copyout(np.uint16, nbytes=M * N * 2), want.copyout(np.uint16, nbytes=M * N * 2), (a, b)


def test_noalloc_matches_the_allocating_entry_point_twice_in_a_row(dev, oracle):
    cap = lib.mrk_hip_gemm_bf16_noalloc_capacity()
    assert cap == 32 << 20
    # split-K shapes (few output tiles, long K): first a larger product, then a smaller one that
    # reuses the front of the same scratch with fewer, shorter partial tiles
    shapes = [(100, 4096, 4096), (37, 1032, 2048)]
    for M, N, K in shapes:
        assert 0 < lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1) <= cap
    for i, (M, N, K) in enumerate(shapes):
        got, want, (a, b) = _pair(dev, M, N, K, 70 + i)
        assert np.array_equal(got, want), (M, N, K)
        if i == 1:  # and against the oracle, at the GEMM tolerance of the other tests
            ref = synth.from_bf16(oracle.gemm_bf16(a, b)).ravel()
            assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # one row against a weight matrix, then back to the first shape: stale partials of the calls
    # in between must not leak into the result
    for M, N, K in [(1, 4096, 4096), (100, 4096, 4096)]:
        got, want, _ = _pair(dev, M, N, K, 80 + M)
        assert np.array_equal(got, want), (M, N, K)


def test_noalloc_unsplit_shapes_and_no_allocator_traffic(dev):
    # shapes with enough tiles use no scratch at all; ragged edges and the any-shape kernel included
    for M, N, K in [(512, 512, 256), (300, 1000, 256), (33, 7, 19)]:
        assert lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1) == 0
        got, want, _ = _pair(dev, M, N, K, 90)
        assert np.array_equal(got, want), (M, N, K)
    # the allocating entry point takes its scratch from the device allocator and parks it in the
    # LRU cache afterwards; the no-alloc one must leave the allocator untouched
    M, N, K = 64, 2048, 4096
    ws = lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    assert ws > 0
    a = morok_amd.Buffer.from_numpy(synth.normal_bf16((M, K), 95, 0), dev.device_id)
    b = morok_amd.Buffer.from_numpy(synth.normal_bf16((K, N), 95, 1), dev.device_id)
    c = dev.buffer(M * N * 2)
    c.ensure_allocated()
    dev.lru_clear()
    ops.gemm_bf16_noalloc(a, b, c, M, N, K, dev.device_id)
    dev.synchronize()
    assert dev.lru_cache_count(ws) == 0 and dev.lru_total_cached() == 0
    ops.gemm_bf16(a, b, c, M, N, K, dev.device_id)
    assert dev.lru_cache_count(ws) == 1


def test_noalloc_argument_errors(dev):
    a = dev.buffer(64)
    with pytest.raises(MorokHipError) as e:  # a device that was never created is not created here
        morok_amd._ffi.check(lib.mrk_hip_gemm_bf16_noalloc(7, a.ptr, a.ptr, a.ptr, 4, 4, 2))
    assert "has not been created" in str(e.value)
    with pytest.raises(MorokHipError):
        morok_amd._ffi.check(lib.mrk_hip_gemm_bf16_noalloc(0, None, a.ptr, a.ptr, 4, 4, 2))
    morok_amd._ffi.check(lib.mrk_hip_gemm_bf16_noalloc(0, None, None, None, 0, 4, 2))  # empty product: nothing to do
