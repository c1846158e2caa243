"""A handful of rows against a Linear layer's weight as it is stored ([out_features, in_features],
tensor/src/nn/linear.rs:9-14,39-41: y = x @ weight.T): the streaming kernels behind
mrk_hip_gemm_bf16_nt / mrk_hip_gemm_f16_nt for M <= 64 (one and two rows on the vector ALUs, 3 to 64 on the
matrix pipes), against the CPU oracle (exact products, f32
accumulate, one rounding) on identical seeded inputs.  Tolerance from the north star: <= 2e-2 max
relative error (max|gpu - ref| / max|ref|) plus the elementwise bound of the tiled kernels' tests
(the result's own rounding plus summation-order noise); against the tiled kernel on the transposed
weight the results may differ by one rounding of the result."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, synth

pytestmark = pytest.mark.gpu

@pytest.fixture()
def T(dev):
    from morok_amd import tensor

    yield tensor
    tensor.set_fusion(True)


SHAPES = [(1, 4096, 4096), (1, 8, 8), (2, 1020, 64), (3, 37, 520), (4, 1024, 4096), (5, 4099, 512), (7, 256, 11008),
          (8, 2048, 2048), (9, 130, 1032), (13, 515, 264), (16, 4096, 1024), (16, 3, 8),
          # every block count of A (1-4) and of the weight (1, 2, 3, 4, 6 blocks per workgroup), K with a partial chunk
          (17, 8192, 1096), (24, 12288, 512), (32, 16384, 264), (33, 22016, 256), (40, 5000, 1032), (48, 24576, 128),
          (49, 4096, 4096), (64, 16384, 520), (64, 77, 40), (61, 12288, 64), (3, 22016, 72), (20, 1, 8)]


def _check(cf, rf, K, ulp):
    assert np.all(np.isfinite(cf))
    scale = np.abs(rf).max()
    assert np.abs(cf - rf).max() <= 2e-2 * scale
    assert np.all(np.abs(cf - rf) <= np.abs(rf) * ulp + 1e-5 * np.sqrt(K) * max(scale / np.sqrt(K), 1.0))


def _run(dev, a16, bt16, nan, f16):
    """a16 [M, K], bt16 [N, K] as uint16 bit patterns; NaNs right behind every operand and the result."""
    M, K = a16.shape
    N = bt16.shape[0]
    pad = np.full(4096, nan, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a16.reshape(-1), pad]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([bt16.reshape(-1), pad]), dev.device_id)
    bc = dev.buffer((M * N + 2048) * 2)
    bc.copyin(np.full(M * N + 2048, nan, np.uint16))
    # as a plan item: up to 64 rows take the streaming kernels and no scratch buffer
    morok_amd.Program.builtin("gemm_f16_nt" if f16 else "gemm_bf16_nt", [M, N, K], dev.device_id).execute([bc, ba, bb])
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == nan)            # nothing written past the result
    return out[: M * N].reshape(M, N), ba, bb


@pytest.mark.parametrize("shape", SHAPES)
def test_skinny_bf16_vs_oracle_and_tiled_kernel(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 13, 0)
    b = synth.normal_bf16((K, N), 13, 1)
    bt = np.ascontiguousarray(b.T)
    got, ba, bb = _run(dev, a, bt, 0x7FC0, False)
    ref = oracle.gemm_bf16(a, b)
    _check(synth.from_bf16(got), synth.from_bf16(ref), K, 2**-7)
    # the tiled kernel on the [K, N] copy sums in another order: the same values up to the result's rounding
    bb2 = morok_amd.Buffer.from_numpy(b, dev.device_id)
    bc2 = dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb2, bc2, M, N, K, dev.device_id)
    tiled = synth.from_bf16(bc2.copyout(np.uint16, (M, N)))
    g = synth.from_bf16(got)
    assert np.all(np.abs(g - tiled) <= np.abs(tiled) * 2**-7 + 2e-5 * np.sqrt(K) * max(np.abs(tiled).max() / np.sqrt(K), 1.0))
    # again: the same bits every time (no atomics, fixed summation order)
    bc3 = dev.buffer(M * N * 2)
    morok_amd.Program.builtin("gemm_bf16_nt", [M, N, K], dev.device_id).execute([bc3, ba, bb])
    assert np.array_equal(bc3.copyout(np.uint16, (M, N)), got)
    # through the ABI: the same kernel
    ops.gemm_bf16_nt(ba, bb, bc3, M, N, K, dev.device_id)
    assert np.array_equal(bc3.copyout(np.uint16, (M, N)), got)


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (3, 37, 520), (8, 2048, 2048), (16, 1000, 1032), (6, 4099, 64), (2, 515, 264),
                                   (24, 12288, 520), (40, 16384, 128), (64, 4100, 1032), (33, 32000, 64)])
def test_skinny_f16_vs_oracle(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal((M, K), 13, 2).astype(np.float16)
    b = synth.normal((K, N), 13, 3).astype(np.float16)
    bt = np.ascontiguousarray(b.T)
    got, _, _ = _run(dev, a.view(np.uint16), bt.view(np.uint16), 0x7E00, True)
    ref = oracle.gemm_f16(a, b)
    _check(got.view(np.float16).astype(np.float32), ref.astype(np.float32), K, 2**-10)


def test_skinny_exact_cases(dev):
    """Values whose sums are exact in f32 whatever the order: small integers.  Every output must be the
    integer dot product, for every row count the kernel is instantiated for and the ones between."""
    rng = np.random.default_rng(5)
    for M in list(range(1, 18)) + [31, 32, 33, 47, 48, 49, 63, 64]:
        N, K = 260 + M, 1544
        a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
        bt = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
        got, _, _ = _run(dev, synth.to_bf16(a), synth.to_bf16(bt), 0x7FC0, False)
        want = a.astype(np.int64) @ bt.astype(np.int64).T            # |sum| <= 16 * 1544 < 2^15: but bf16 keeps 8 bits
        assert np.array_equal(got, synth.to_bf16(want.astype(np.float32)))


def test_skinny_batched_plan_item(dev, oracle):
    """{M, N, K, batch}: that many products over operands stored back to back."""
    for M, N, K, B in ((4, 520, 1024, 3), (2, 130, 512, 2), (20, 4100, 264, 3)):
        _batched(dev, oracle, M, N, K, B)


def _batched(dev, oracle, M, N, K, B):
    a = synth.normal_bf16((B, M, K), 13, 4)
    bt = synth.normal_bf16((B, N, K), 13, 5)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(bt, dev.device_id)
    bc = dev.buffer(B * M * N * 2)
    morok_amd.Program.builtin("gemm_bf16_nt", [M, N, K, B], dev.device_id).execute([bc, ba, bb])
    got = bc.copyout(np.uint16, (B, M, N))
    for i in range(B):
        ref = oracle.gemm_bf16(a[i], np.ascontiguousarray(bt[i].T))
        _check(synth.from_bf16(got[i]), synth.from_bf16(ref), K, 2**-7)


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (2, 1020, 64), (5, 37, 520), (16, 4096, 1024), (33, 515, 264), (64, 12288, 512)])
def test_streamed_residual_add(dev, shape):
    """h + x @ w.T for a handful of rows, as the plan item the scheduler picks ("gemm_bf16_nt_residual"): the
    streaming kernels add h where they write their result, with the bits of the product followed by the add."""
    M, N, K = shape
    x, w, h = synth.normal_bf16((M, K), 13, 30), synth.normal_bf16((N, K), 13, 31), synth.normal_bf16((M, N), 13, 32)
    bx, bw, bh = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (x, w, h))
    by = dev.buffer((M * N + 2048) * 2)
    by.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    morok_amd.Program.builtin("gemm_bf16_nt_residual", [M, N, K], dev.device_id).execute([by, bx, bw, bh])
    out = by.copyout(np.uint16)
    assert np.all(out[M * N:] == 0x7FC0)
    bp = dev.buffer(M * N * 2)
    ops.gemm_bf16_nt(bx, bw, bp, M, N, K, dev.device_id)
    want = synth.to_bf16(synth.from_bf16(bp.copyout(np.uint16, (M, N))) + synth.from_bf16(h))
    assert np.array_equal(out[: M * N].reshape(M, N), want)


def test_linear_decode_with_residual_is_one_kernel(T, oracle):
    """h + x.linear(w) over 8 rows: one streaming kernel (no elementwise kernel behind it), the bits of the unfused pair."""
    from morok_amd import uop

    M, K, N = 8, 1024, 3072
    x, w, h = synth.normal_bf16((M, K), 13, 33), synth.normal_bf16((N, K), 13, 34), synth.normal_bf16((M, N), 13, 35)
    tx, tw, th = (T.Tensor.from_numpy(t, uop.BF16) for t in (x, w, h))
    T.set_fusion(True)
    r = th.try_add(tx.linear(tw))
    got = r.to_numpy()
    assert r.kernels() == [f"gemm_bf16_nt_residual_{M}_{N}_{K}"]
    p = tx.linear(tw).to_numpy()
    assert np.array_equal(got, synth.to_bf16(synth.from_bf16(p) + synth.from_bf16(h)))
    ref = synth.from_bf16(oracle.gemm_bf16(x, np.ascontiguousarray(w.T))) + synth.from_bf16(h)
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()


@pytest.mark.parametrize("shape", [(1, 4096, 1024), (4, 1024, 512), (16, 11008, 4096), (33, 520, 264), (64, 2816, 1024), (7, 136, 72), (48, 4104, 520)])
def test_streamed_gated_product(dev, T, shape):
    """silu(x @ Wg.T) * (x @ Wu.T) over a weight [2F, K] (gate rows first) for a handful of rows: the gated form of the
    streaming kernel ("gemm_bf16_nt_swiglu").  On small-integer data both products are exact, so the result must be
    the generated elementwise kernel's on the exact products, bit for bit; on normal data the two may differ where a
    product's f32 sum rounds the other way (another summation order), i.e. by roundings of single elements."""
    from morok_amd import uop

    M, F, K = shape
    rng = np.random.default_rng(11)
    for exact in (True, False):
        if exact:
            x = synth.to_bf16(rng.integers(-2, 3, size=(M, K)).astype(np.float32))
            w = synth.to_bf16(rng.integers(-2, 3, size=(2 * F, K)).astype(np.float32))
        else:
            x, w = synth.normal_bf16((M, K), 13, 40), (synth.from_bf16(synth.normal_bf16((2 * F, K), 13, 41)) / np.sqrt(K)).astype(np.float32)
            w = synth.to_bf16(w)
        bx, bw = morok_amd.Buffer.from_numpy(x, dev.device_id), morok_amd.Buffer.from_numpy(w, dev.device_id)
        bg = dev.buffer((M * F + 2048) * 2)
        bg.copyin(np.full(M * F + 2048, 0x7FC0, np.uint16))
        morok_amd.Program.builtin("gemm_bf16_nt_swiglu", [M, F, K], dev.device_id).execute([bg, bx, bw])
        out = bg.copyout(np.uint16)
        assert np.all(out[M * F:] == 0x7FC0)
        got = out[: M * F].reshape(M, F)
        # the unfused pair: the packed product, then the generated kernel over its two halves
        bp = dev.buffer(M * 2 * F * 2)
        ops.gemm_bf16_nt(bx, bw, bp, M, 2 * F, K, dev.device_id)
        p = T.Tensor.from_numpy(bp.copyout(np.uint16, (M, 2 * F)), uop.BF16)
        want = p.try_shrink([(0, M), (0, F)]).silu().try_mul(p.try_shrink([(0, M), (F, 2 * F)])).to_numpy()
        if exact:
            assert np.array_equal(got, want)
        else:
            g, wv = synth.from_bf16(got), synth.from_bf16(want)
            assert np.all(np.isfinite(g))
            assert np.mean(got == want) >= 0.97
            assert np.all(np.abs(g - wv) <= np.abs(wv) * 2.0 ** -6 + 1e-3 * np.abs(wv).max())


def test_linear_decode_gate_is_one_kernel(T, oracle):
    """The gated feed-forward half of a decode step over Linear-layout weights: one streaming kernel."""
    from morok_amd import uop

    M, K, F = 8, 1024, 1536
    x, w13 = synth.normal_bf16((M, K), 13, 42), synth.normal_bf16((2 * F, K), 13, 43)
    tx, tw = T.Tensor.from_numpy(x, uop.BF16), T.Tensor.from_numpy(w13, uop.BF16)
    T.set_fusion(True)
    gu = tx.linear(tw)
    g = gu.try_shrink([(0, M), (0, F)]).silu().try_mul(gu.try_shrink([(0, M), (F, 2 * F)]))
    got = g.to_numpy()
    assert g.kernels() == [f"gemm_bf16_nt_swiglu_{M}_{F}_{K}"]
    ref = oracle.gemm_bf16(x, np.ascontiguousarray(w13.T))
    gate, up = synth.from_bf16(ref[:, :F]), synth.from_bf16(ref[:, F:])
    with np.errstate(over="ignore"):
        want = gate / (1.0 + np.exp(-gate)) * up
    assert np.abs(synth.from_bf16(got) - want).max() <= 2e-2 * np.abs(want).max()


def test_skinny_refusals(dev):
    a, b, c = dev.buffer(72 * 4096 * 2), dev.buffer(4096 * 1024 * 2), dev.buffer(72 * 1024 * 2)
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_nt(a, b, c, 4, 1024, 4092, dev.device_id)    # K not a multiple of 8
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_nt(a, b, c, 65, 1020, 4096, dev.device_id)   # more than 64 rows and N not a multiple of 8


def test_linear_decode_step_is_one_kernel(T, oracle):
    """x [1, K] (and batches of 8, 12 and 64) through Tensor.linear with the weight as stored: one product that
    reads the weight in place, no transposed copy, no scratch (up to 64 rows stream it in one pass; 80 take the
    tiled kernels with the K loop spread over the chip)."""
    from morok_amd import uop

    T.set_fusion(True)
    K, N = 2048, 3072
    w = synth.normal_bf16((N, K), 13, 6)
    tw = T.Tensor.from_numpy(w, uop.BF16)
    for M in (1, 8, 12, 64, 80):
        x = synth.normal_bf16((M, K), 13, 7)
        y = T.Tensor.from_numpy(x, uop.BF16).linear(tw)
        got = y.to_numpy()
        assert y.kernels() == [f"gemm_bf16_nt_{M}_{N}_{K}" + ("" if M <= 64 else "_splitk")]
        ref = oracle.gemm_bf16(x, np.ascontiguousarray(w.T))
        _check(synth.from_bf16(got), synth.from_bf16(ref), K, 2**-7)


# ---------------------------------------------------------------- the same rows against a weight stored [K, N]
KN_SHAPES = [(1, 4096, 4096), (1, 520, 1024), (1, 264, 4104), (1, 12288, 4096), (1, 1024, 256), (1, 256, 11008), (1, 4104, 520),
             (1, 8, 4096), (1, 2048, 2048), (1, 24576, 512)]


@pytest.mark.parametrize("shape", KN_SHAPES)
def test_skinny_kn_form_vs_oracle_and_tiled_kernel(dev, oracle, shape):
    """One row through mrk_hip_gemm_bf16 ([K, N] weight): one streaming pass on the vector ALUs into f32 partial sums
    plus their sum.  Against the oracle, against the tiled kernel (another summation order), the
    same bits on every run, through the ABI (allocator scratch) and as a plan item with a scratch buffer;
    NaNs right behind the operands and the result show that nothing reads or writes past them."""
    from morok_amd._ffi import lib

    M, N, K = shape
    ws = lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    assert ws > 0 and ws % (M * N * 4) == 0
    a = synth.normal_bf16((M, K), 13, 8)
    b = synth.normal_bf16((K, N), 13, 9)
    pad = np.full(4096, 0x7FC0, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.reshape(-1), pad]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([b.reshape(-1), pad]), dev.device_id)
    bc = dev.buffer((M * N + 2048) * 2)
    bc.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == 0x7FC0)
    got = out[: M * N].reshape(M, N)
    ref = oracle.gemm_bf16(a, b)
    _check(synth.from_bf16(got), synth.from_bf16(ref), K, 2**-7)
    bc2 = dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, bc2, M, N, K, dev.device_id, 4)          # the tiled kernel, unsplit
    tiled = synth.from_bf16(bc2.copyout(np.uint16, (M, N)))
    g = synth.from_bf16(got)
    assert np.all(np.abs(g - tiled) <= np.abs(tiled) * 2**-7 + 2e-5 * np.sqrt(K) * max(np.abs(tiled).max() / np.sqrt(K), 1.0))
    ops.gemm_bf16(ba, bb, bc2, M, N, K, dev.device_id)
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)
    bw = dev.buffer(ws + 4096)
    bw.copyin(np.full((ws + 4096) // 4, np.nan, np.float32))
    prog = morok_amd.Program.builtin("gemm_bf16", [M, N, K, 1, ws], dev.device_id)
    prog.execute([bc2, ba, bb, bw])
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)
    assert np.all(np.isnan(bw.copyout(np.float32)[ws // 4:]))     # the partial sums stay inside the scratch asked for


ROWS_KN_SHAPES = [(3, 4096, 4096), (16, 12288, 4096), (8, 520, 1024), (5, 264, 4104), (16, 22016, 512), (12, 8, 4096),
                  (16, 32000, 256), (4, 1024, 264), (7, 8200, 2056), (9, 4096, 11008), (16, 72, 296),
                  # two rows; one row against more than 24576 columns; 17 to 64 rows against a narrow weight
                  (2, 520, 1024), (2, 12288, 4096), (2, 256, 11008), (2, 8, 4096), (2, 24576, 512), (1, 32000, 1024),
                  (17, 4096, 4096), (33, 1032, 8192), (48, 264, 2056), (64, 4096, 4096), (40, 4096, 296)]


@pytest.mark.parametrize("shape", ROWS_KN_SHAPES)
def test_rows_kn_form_vs_oracle_and_tiled_kernel(dev, oracle, shape):
    """2 to 16 rows (to 64 against a narrow weight) through mrk_hip_gemm_bf16 ([K, N] weight): the weight streamed once through LDS and the
    transposing read onto the matrix pipes, f32 partial sums per K range plus their sum (or one launch when one
    range is enough).  Against the oracle, against the tiled kernel (another summation order), the same bits
    on every run, through the ABI and as a plan item; NaNs right behind the operands, the result and the scratch."""
    from morok_amd._ffi import lib

    M, N, K = shape
    ws = lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    assert ws % (M * N * 4) == 0 and ws <= 32 << 20
    a = synth.normal_bf16((M, K), 13, 14)
    b = synth.normal_bf16((K, N), 13, 15)
    pad = np.full(4096, 0x7FC0, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.reshape(-1), pad]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([b.reshape(-1), pad]), dev.device_id)
    bc = dev.buffer((M * N + 2048) * 2)
    bc.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == 0x7FC0)
    got = out[: M * N].reshape(M, N)
    _check(synth.from_bf16(got), synth.from_bf16(oracle.gemm_bf16(a, b)), K, 2**-7)
    bc2 = dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, bc2, M, N, K, dev.device_id, 4)          # the tiled kernel, unsplit
    tiled = synth.from_bf16(bc2.copyout(np.uint16, (M, N)))
    g = synth.from_bf16(got)
    assert np.all(np.abs(g - tiled) <= np.abs(tiled) * 2**-7 + 2e-5 * np.sqrt(K) * max(np.abs(tiled).max() / np.sqrt(K), 1.0))
    ops.gemm_bf16(ba, bb, bc2, M, N, K, dev.device_id)
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)
    if ws:
        bw = dev.buffer(ws + 4096)
        bw.copyin(np.full((ws + 4096) // 4, np.nan, np.float32))
        morok_amd.Program.builtin("gemm_bf16", [M, N, K, 1, ws], dev.device_id).execute([bc2, ba, bb, bw])
        assert np.all(np.isnan(bw.copyout(np.float32)[ws // 4:]))     # the partial sums stay inside the scratch asked for
    else:
        morok_amd.Program.builtin("gemm_bf16", [M, N, K], dev.device_id).execute([bc2, ba, bb])
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)


def test_skinny_kn_form_f16_and_exact(dev, oracle):
    M, N, K = 4, 1032, 2048
    a = synth.normal((M, K), 13, 10).astype(np.float16)
    b = synth.normal((K, N), 13, 11).astype(np.float16)
    ba, bb = morok_amd.Buffer.from_numpy(a.view(np.uint16), dev.device_id), morok_amd.Buffer.from_numpy(b.view(np.uint16), dev.device_id)
    bc = dev.buffer(M * N * 2)
    ops.gemm_f16(ba, bb, bc, M, N, K, dev.device_id)
    got = bc.copyout(np.uint16, (M, N)).view(np.float16).astype(np.float32)
    _check(got, oracle.gemm_f16(a, b).astype(np.float32), K, 2**-10)
    # small integers: every sum is exact in f32 whatever the order (up to 16 rows stream, more take the tiles)
    rng = np.random.default_rng(6)
    for M in list(range(1, 18)) + [33]:
        N, K = 520 + 8 * M, 1288
        ai = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
        bi = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
        ba, bb = morok_amd.Buffer.from_numpy(synth.to_bf16(ai), dev.device_id), morok_amd.Buffer.from_numpy(synth.to_bf16(bi), dev.device_id)
        bc = dev.buffer(M * N * 2)
        ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id)
        want = ai.astype(np.int64) @ bi.astype(np.int64)
        assert np.array_equal(bc.copyout(np.uint16, (M, N)), synth.to_bf16(want.astype(np.float32)))


def test_matmul_decode_step_kn_weight(T, oracle):
    """x [M, K] @ w [K, N] through Tensor.matmul for a handful of rows: one plan item with scratch placed by
    the plan (the streaming kernels: one row on the vector ALUs, eight on the matrix pipes; K split over the chip)."""
    from morok_amd import uop

    T.set_fusion(True)
    K, N = 2048, 3072
    w = synth.normal_bf16((K, N), 13, 12)
    tw = T.Tensor.from_numpy(w, uop.BF16)
    for M in (1, 8):
        x = synth.normal_bf16((M, K), 13, 13)
        y = T.Tensor.from_numpy(x, uop.BF16).matmul(tw)
        got = y.to_numpy()
        assert y.kernels() == [f"gemm_bf16_{M}_{N}_{K}_splitk"]
        _check(synth.from_bf16(got), synth.from_bf16(oracle.gemm_bf16(x, w)), K, 2**-7)


@pytest.mark.parametrize("seed", range(6))
def test_skinny_random_shapes_exact(dev, seed):
    """Random shapes on small-integer data, where every sum is exact in f32 whatever its order: the
    [N, K] form for 1-64 rows (any N, K a multiple of 8; now and then with a bias row or a residual matrix of small
    integers, whose sum with the product is exact as well) and the [K, N] form for 1-64 rows (N, K multiples of 8)
    must give the integer results exactly, whichever kernel the shape selects."""
    rng = np.random.default_rng(7000 + seed)
    for it in range(12):
        M = int(rng.integers(1, 65)) if it % 3 else int(rng.integers(1, 17))
        N = int(rng.integers(1, 700)) if it % 4 else int(rng.integers(1, 400)) * 16 + int(rng.integers(0, 16))
        K = 8 * int(rng.integers(1, 300))
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        bt = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
        want = synth.to_bf16((a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32))
        ba, bb = morok_amd.Buffer.from_numpy(synth.to_bf16(a), dev.device_id), morok_amd.Buffer.from_numpy(synth.to_bf16(bt), dev.device_id)
        bc = dev.buffer(M * N * 2)
        morok_amd.Program.builtin("gemm_bf16_nt", [M, N, K], dev.device_id).execute([bc, ba, bb])
        assert np.array_equal(bc.copyout(np.uint16, (M, N)), want), (M, N, K)
        if it % 2:
            # |product| <= 9 K and the addend keep the sum an integer below 2^24; the result is rounded once more to bf16
            row = bool(rng.integers(0, 2))
            add = rng.integers(-3, 4, size=(N,) if row else (M, N)).astype(np.float32)
            badd = morok_amd.Buffer.from_numpy(synth.to_bf16(add), dev.device_id)
            morok_amd.Program.builtin("gemm_bf16_nt_bias" if row else "gemm_bf16_nt_residual", [M, N, K], dev.device_id).execute([bc, ba, bb, badd])
            want_add = synth.to_bf16(synth.from_bf16(want) + add)
            assert np.array_equal(bc.copyout(np.uint16, (M, N)), want_add), (M, N, K, row)
        N8 = 8 * int(rng.integers(1, 200))
        K2 = 8 * int(rng.integers(32, 400))
        a2 = rng.integers(-3, 4, size=(M, K2)).astype(np.float32)
        b2 = rng.integers(-3, 4, size=(K2, N8)).astype(np.float32)
        want2 = synth.to_bf16((a2.astype(np.int64) @ b2.astype(np.int64)).astype(np.float32))
        ba2, bb2 = morok_amd.Buffer.from_numpy(synth.to_bf16(a2), dev.device_id), morok_amd.Buffer.from_numpy(synth.to_bf16(b2), dev.device_id)
        bc2 = dev.buffer(M * N8 * 2)
        ops.gemm_bf16(ba2, bb2, bc2, M, N8, K2, dev.device_id)
        assert np.array_equal(bc2.copyout(np.uint16, (M, N8)), want2), (M, N8, K2)
