"""Parity of the hand-written half-precision (f16) GEMM with the CPU oracle (exact f16 x f16
products, f32 accumulate along k, one rounding to f16) on identical seeded inputs: the f16
instantiation of the tiled kernels around v_mfma_f32_16x16x32_f16 (the f16 entry of the
reference's CDNA4 tensor-core table, schedule/src/optimizer/renderer.rs:724-733).  Tolerance
from the north star: <= 2e-2 max relative error (max|gpu - ref| / max|ref|); a tighter
elementwise bound (one f16 ulp plus summation-order noise) is asserted as well."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, synth

pytestmark = pytest.mark.gpu
NAN16 = 0x7E00


def _inputs(M, N, K, tid):
    return synth.normal((M, K), 5, tid).astype(np.float16), synth.normal((K, N), 5, tid + 1).astype(np.float16)


def _gemm(dev, a, b, kind="abi"):
    M, K = a.shape
    N = b.shape[1]
    ba = morok_amd.Buffer.from_numpy(a.view(np.uint16), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(b.view(np.uint16), dev.device_id)
    bc = dev.buffer(max(M * N * 2, 1))
    if kind == "program":
        morok_amd.Program.builtin("gemm_f16", [M, N, K], dev.device_id).execute([bc, ba, bb])
    else:
        ops.gemm_f16(ba, bb, bc, M, N, K, dev.device_id)
    return bc.copyout(np.uint16, nbytes=M * N * 2).reshape(M, N).view(np.float16)


def _check(c, ref, K):
    cf, rf = c.astype(np.float32), ref.astype(np.float32)
    assert np.all(np.isfinite(cf))
    scale = np.abs(rf).max()
    assert np.abs(cf - rf).max() <= 2e-2 * scale
    assert np.all(np.abs(cf - rf) <= np.abs(rf) * 2**-10 + 1e-5 * np.sqrt(K) * max(scale / np.sqrt(K), 1.0))


@pytest.mark.parametrize("shape", [(256, 256, 64), (256, 512, 128), (512, 256, 1024), (768, 1024, 192), (256, 256, 320),
                                   (1, 8, 64), (37, 264, 128), (257, 520, 64), (1000, 776, 320),             # ragged M / N
                                   (256, 256, 8), (256, 256, 72), (100, 264, 200), (512, 512, 1000)])         # ragged K
def test_gemm_f16_tiled_kernels_vs_oracle(dev, oracle, shape):
    M, N, K = shape
    a, b = _inputs(M, N, K, 0)
    got = _gemm(dev, a, b)
    _check(got, oracle.gemm_f16(a, b), K)
    assert np.array_equal(got.view(np.uint16), _gemm(dev, a, b, "program").view(np.uint16))


@pytest.mark.parametrize("shape", [(1, 1, 1), (33, 65, 17), (100, 200, 300), (5, 7, 1000), (64, 12, 64), (130, 256, 20)])
def test_gemm_f16_any_shape_kernel(dev, oracle, shape):
    """N or K not a multiple of 8: the one-wave-per-tile kernel, same products."""
    M, N, K = shape
    a, b = _inputs(M, N, K, 2)
    _check(_gemm(dev, a, b), oracle.gemm_f16(a, b), K)


def test_gemm_f16_exact_cases_and_no_stray_accesses(dev):
    M, N, K = 300, 264, 200
    a, b = _inputs(M, N, K, 4)
    nan = np.full(8192, NAN16, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.view(np.uint16).reshape(-1), nan]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([b.view(np.uint16).reshape(-1), nan]), dev.device_id)
    bc = dev.buffer(M * N * 2 + 4096)
    bc.copyin(np.full(M * N + 2048, NAN16, np.uint16))
    ops.gemm_f16(ba, bb, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == NAN16)                                   # nothing written past C
    assert np.array_equal(out[: M * N].reshape(M, N), _gemm(dev, a, b).view(np.uint16))   # nothing read past A / B
    eye = np.eye(256, dtype=np.float16)
    x = synth.normal((256, 256), 5, 9).astype(np.float16)
    assert np.array_equal(_gemm(dev, x, eye).view(np.uint16), x.view(np.uint16))
    assert np.array_equal(_gemm(dev, eye, x).view(np.uint16), x.view(np.uint16))
    small = (synth.uniform((128, 512), 5, 10) * 4).astype(np.int32).astype(np.float16)
    ones = np.ones((512, 64), np.float16)
    assert np.array_equal(_gemm(dev, small, ones).astype(np.float64), small.astype(np.float64).sum(1, keepdims=True).repeat(64, 1))
    # f16 has no headroom beyond 65504: a product that overflows comes out as infinity, as the oracle's does
    big = np.full((64, 64), 200.0, np.float16)
    assert np.isinf(_gemm(dev, big, big)).all()


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (16, 1024, 2048), (100, 264, 4000), (37, 2048, 4096)])
def test_gemm_f16_split_k(dev, oracle, shape):
    from morok_amd._ffi import lib

    M, N, K = shape
    ws = lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    assert ws > 0
    a, b = _inputs(M, N, K, 6)
    got = _gemm(dev, a, b)
    _check(got, oracle.gemm_f16(a, b), K)
    assert np.array_equal(got.view(np.uint16), _gemm(dev, a, b).view(np.uint16))        # the same bits on every run
    ba, bb = morok_amd.Buffer.from_numpy(a.view(np.uint16), dev.device_id), morok_amd.Buffer.from_numpy(b.view(np.uint16), dev.device_id)
    bc, bw = dev.buffer(M * N * 2), dev.buffer(ws)
    prog = morok_amd.Program.builtin("gemm_f16", [M, N, K, 1, ws], dev.device_id)
    assert prog.name.endswith("_splitk")
    prog.execute([bc, ba, bb, bw])
    assert np.array_equal(bc.copyout(np.uint16, (M, N)), got.view(np.uint16))


@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 256), (300, 520, 128), (1000, 776, 320), (256, 256, 72), (2048, 512, 136)])
def test_gemm_f16_transposed_second_operand(dev, oracle, shape):
    """a @ bt.T with bt [N, K] read in place (a Linear layer's weight): the same products in the
    same order as the [K, N] form, so the same bits."""
    M, N, K = shape
    a, b = _inputs(M, N, K, 8)
    bt = np.ascontiguousarray(b.T)
    ba = morok_amd.Buffer.from_numpy(a.view(np.uint16), dev.device_id)
    bbt = morok_amd.Buffer.from_numpy(bt.view(np.uint16), dev.device_id)
    bc = dev.buffer(M * N * 2)
    ops.gemm_f16_nt(ba, bbt, bc, M, N, K, dev.device_id)
    got = bc.copyout(np.uint16, (M, N))
    _check(got.view(np.float16), oracle.gemm_f16(a, b), K)
    assert np.array_equal(got, _gemm(dev, a, b).view(np.uint16))
    bc2 = dev.buffer(M * N * 2)
    morok_amd.Program.builtin("gemm_f16_nt", [M, N, K], dev.device_id).execute([bc2, ba, bbt])
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)


def test_gemm_f16_full_size_rows_and_linearity(dev, oracle):
    """4096^3 (the bf16 headline shape, in half precision): sampled rows against the oracle, and
    (2A) B == 2 (A B) exactly where nothing overflows."""
    M = N = K = 4096
    a, b = _inputs(M, N, K, 10)
    a = (a * np.float16(0.25)).astype(np.float16)
    c = _gemm(dev, a, b)
    rows = np.array([0, 1, 255, 256, 1000, 2047, 2048, 4095])
    _check(c[rows], oracle.gemm_f16(np.ascontiguousarray(a[rows]), b), K)
    c2 = _gemm(dev, (a * np.float16(2)).astype(np.float16), b)
    cf, c2f = c.astype(np.float32), c2.astype(np.float32)
    normal = np.abs(cf) >= 2.0 ** -13                       # results in f16's subnormal range round on a coarser grid than their doubles
    assert np.array_equal(c2f[normal], cf[normal] * 2)
    assert np.abs(c2f[~normal] - cf[~normal] * 2).max() <= 2.0 ** -24


def test_gemm_f16_agrees_with_the_generated_tensor_core_kernel(dev):
    """The WMMA route of the same product (f16 16x16x32 tensor core, register-only generated
    kernel) adds the same products in the same order: the same bits."""
    from morok_amd import sched, uop as U

    M, N, K = 256, 192, 128
    a, b = _inputs(M, N, K, 12)
    spec = U.render(sched.build_wmma_matmul(2, M, N, K, U.F16), "r_tc_h_vs_hand", dev.device_id)
    prog = morok_amd.Program.create(morok_amd.compile_spec(spec), dev.device_id)
    ba, bb = morok_amd.Buffer.from_numpy(a.view(np.uint16), dev.device_id), morok_amd.Buffer.from_numpy(b.view(np.uint16), dev.device_id)
    bc = dev.buffer(M * N * 2)
    prog.execute([bc, ba, bb], ())
    assert np.array_equal(bc.copyout(np.uint16, (M, N)), _gemm(dev, a, b).view(np.uint16))
