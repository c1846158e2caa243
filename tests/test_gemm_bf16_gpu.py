"""Parity of the MFMA bf16 GEMM with the CPU oracle (exact products, f32 accumulate, one
rounding to bf16) on identical seeded inputs.  Tolerance from the north star: <= 2e-2 max
relative error, measured as max|gpu - ref| / max|ref|; a tighter elementwise bound
(2 bf16 ulps of the result plus summation-order noise) is asserted as well."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, synth

pytestmark = pytest.mark.gpu


def _gemm(dev, a, b, variant=0, via_program=False):
    M, K = a.shape
    N = b.shape[1]
    ba = morok_amd.Buffer.from_numpy(a, dev.device_id)
    bb = morok_amd.Buffer.from_numpy(b, dev.device_id)
    bc = dev.buffer(max(M * N * 2, 1))
    if via_program:
        morok_amd.Program.builtin("gemm_bf16", [M, N, K], dev.device_id).execute([bc, ba, bb])
    else:
        ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id, variant)
    return bc.copyout(np.uint16, nbytes=M * N * 2).reshape(M, N)


def _check(c, ref, K):
    cf, rf = synth.from_bf16(c), synth.from_bf16(ref)
    assert np.all(np.isfinite(cf))
    scale = np.abs(rf).max()
    assert np.abs(cf - rf).max() <= 2e-2 * scale
    # f32 accumulation order differs between MFMA and the sequential oracle: error of the
    # f32 sum ~ K * 2^-24 * sqrt(K), then one bf16 rounding each (they may round apart by 1 ulp)
    assert np.all(np.abs(cf - rf) <= np.abs(rf) * 2**-7 + 1e-5 * np.sqrt(K) * max(scale / np.sqrt(K), 1.0))


# K / 64 = 1, 2, 16, 3, 5, 6, 7 steps: the pipeline cycles three B stages and two A stages and is
# unrolled by two, so short, odd and even step counts take different paths through it
@pytest.mark.parametrize("shape", [(256, 256, 64), (256, 512, 128), (512, 256, 1024), (768, 1024, 192),
                                   (256, 256, 320), (512, 512, 384), (256, 512, 448)])
def test_gemm_tiled_kernel_parity(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 0)
    b = synth.normal_bf16((K, N), 3, 1)
    _check(_gemm(dev, a, b), oracle.gemm_bf16(a, b), K)


# ragged M (any) and N (whole 16-byte chunks) run the tiled kernel with redirected edge loads
# and masked stores; the last tile row / column may be almost empty or almost full
@pytest.mark.parametrize("shape", [(1, 8, 64), (37, 264, 128), (255, 248, 192), (257, 520, 64), (300, 1000, 256),
                                   (513, 256, 128), (256, 8, 64), (1000, 776, 320)])
def test_gemm_tiled_kernel_ragged_edges(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 6)
    b = synth.normal_bf16((K, N), 3, 7)
    got = _gemm(dev, a, b)
    _check(got, oracle.gemm_bf16(a, b), K)
    # the generic kernel agrees bit for bit (same products, same order of the K steps)
    assert np.array_equal(got, _gemm(dev, a, b, variant=2))


# K in whole 16-byte chunks but not in whole 64-deep steps: the last step's out-of-range chunks
# are copied from a block of zeros
@pytest.mark.parametrize("shape", [(256, 256, 8), (256, 256, 72), (100, 264, 200), (512, 512, 1000), (300, 40, 136),
                                   (256, 256, 56), (64, 128, 120)])
def test_gemm_tiled_kernel_ragged_k(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 8)
    b = synth.normal_bf16((K, N), 3, 9)
    got = _gemm(dev, a, b)
    _check(got, oracle.gemm_bf16(a, b), K)
    assert np.array_equal(got, _gemm(dev, a, b, variant=2))


@pytest.mark.parametrize("variant", [3, 4])
@pytest.mark.parametrize("shape", [(256, 256, 72), (256, 256, 64), (300, 264, 128), (100, 8, 200), (255, 1000, 8)])
def test_gemm_does_not_read_past_the_operands(dev, oracle, shape, variant):
    """Edge tiles and the partial last K step must not read beyond A and B: NaNs placed right
    behind them in the same allocations do not reach the result (a stray operand would, even
    against a zero: NaN * 0 = NaN)."""
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 10)
    b = synth.normal_bf16((K, N), 3, 11)
    nan = np.full(8192, 0x7FC0, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.reshape(-1), nan]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([b.reshape(-1), nan]), dev.device_id)
    bc = dev.buffer(M * N * 2 + 4096)
    bc.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id, variant)
    out = bc.copyout(np.uint16)
    _check(out[: M * N].reshape(M, N), oracle.gemm_bf16(a, b), K)
    assert np.all(out[M * N:] == 0x7FC0)   # and nothing is written behind C


# The 128-row tile (chosen by itself when the shape has few tiles) and the 256-row tile are the
# same pipeline: forced either way they agree bit for bit with each other and with the oracle
# within tolerance, on full, ragged-M/N and ragged-K shapes and on a batch.
@pytest.mark.parametrize("shape", [(128, 256, 64), (512, 512, 256), (1000, 776, 320), (100, 264, 200), (384, 1024, 1000),
                                   (129, 8, 72), (2048, 512, 128)])
def test_gemm_both_tile_sizes_agree(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 12)
    b = synth.normal_bf16((K, N), 3, 13)
    big, small = _gemm(dev, a, b, variant=3), _gemm(dev, a, b, variant=4)
    _check(small, oracle.gemm_bf16(a, b), K)
    assert np.array_equal(big, small)
    assert np.array_equal(_gemm(dev, a, b), small)


@pytest.mark.parametrize("shape", [(1, 1, 1), (32, 32, 16), (33, 65, 17), (100, 200, 300), (5, 7, 1000),
                                   (255, 257, 63), (64, 64, 0)])
def test_gemm_generic_kernel_parity(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 2)
    b = synth.normal_bf16((K, N), 3, 3)
    _check(_gemm(dev, a, b), oracle.gemm_bf16(a, b), max(K, 1))


def test_gemm_both_kernels_agree_and_program_path(dev, oracle):
    a = synth.normal_bf16((256, 128), 3, 4)
    b = synth.normal_bf16((128, 256), 3, 5)
    ref = oracle.gemm_bf16(a, b)
    _check(_gemm(dev, a, b, variant=2), ref, 128)
    _check(_gemm(dev, a, b, via_program=True), ref, 128)


def test_gemm_special_cases_exact(dev):
    # identity / permutation / ones: exact in bf16, so bit-for-bit
    n = 256
    a = synth.normal_bf16((n, n), 3, 6)
    eye = synth.to_bf16(np.eye(n, dtype=np.float32))
    assert np.array_equal(_gemm(dev, a, eye), a)
    assert np.array_equal(_gemm(dev, eye, a), a)
    perm = synth.to_bf16(np.eye(n, dtype=np.float32)[:, ::-1].copy())
    assert np.array_equal(_gemm(dev, a, perm), a[:, ::-1])
    ones = synth.to_bf16(np.ones((n, 512), np.float32))
    c = synth.from_bf16(_gemm(dev, ones, synth.to_bf16(np.ones((512, n), np.float32))))
    assert np.all(c == 512)
    # asymmetric operands catch a transposed A or B
    a2 = synth.to_bf16(np.arange(256 * 64, dtype=np.float32).reshape(256, 64) % 7 - 3)
    b2 = synth.to_bf16(np.arange(64 * 256, dtype=np.float32).reshape(64, 256) % 5 - 2)
    ref = synth.from_bf16(a2).astype(np.float64) @ synth.from_bf16(b2).astype(np.float64)
    assert np.array_equal(synth.from_bf16(_gemm(dev, a2, b2)), synth.from_bf16(synth.to_bf16(ref.astype(np.float32))))


def test_gemm_full_size_config_slice_and_linearity(dev, oracle):
    # configs[2] shape 4096^3: rows of the full product against the oracle, plus linearity
    M = N = K = 4096
    a = synth.normal_bf16((M, K), 3, 0)
    b = synth.normal_bf16((K, N), 3, 1)
    c = _gemm(dev, a, b)
    rows = np.array([0, 1, 255, 256, 1000, 2047, 2048, 4095])
    ref = oracle.gemm_bf16(np.ascontiguousarray(a[rows]), b)
    _check(c[rows], ref, K)
    # size-independent property: (2A) B == 2 (A B) exactly (scaling by 2 is exact in bf16 and f32)
    a2 = synth.to_bf16(synth.from_bf16(a) * 2)
    c2 = _gemm(dev, a2, b)
    assert np.array_equal(synth.from_bf16(c2), synth.from_bf16(c) * 2)


@pytest.mark.parametrize("seed", range(24))
def test_gemm_random_shapes(dev, oracle, seed):
    """Random M, N, K (any, including ones that fall back to the any-shape kernel) and a random
    forced variant: all paths agree with the oracle, and the tiled ones with each other."""
    rng = np.random.default_rng(2000 + seed)
    M = int(rng.integers(1, 700))
    N = int(rng.integers(1, 90)) * (8 if seed % 3 else 1)
    K = int(rng.integers(1, 60)) * (8 if seed % 4 else 1)
    a = synth.normal_bf16((M, K), 3, 100 + seed)
    b = synth.normal_bf16((K, N), 3, 200 + seed)
    ref = oracle.gemm_bf16(a, b)
    outs = [_gemm(dev, a, b, variant=v) for v in (0, 2, 3, 4)]
    for o in outs:
        _check(o, ref, K)
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (16, 1024, 2048), (100, 264, 4000), (16, 512, 2056), (37, 2048, 4096)])
def test_gemm_split_k(dev, oracle, shape):
    """Few output tiles against a long K: the K loop is spread over the chip, f32 partials go to
    scratch from the device allocator and are added in a fixed order.  Against the oracle, the
    unsplit kernel (which it may differ from by the rounding of one more f32 addition chain)
    and itself (the same bits on every run)."""
    from morok_amd._ffi import lib

    M, N, K = shape
    assert lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1) > 0
    a = synth.normal_bf16((M, K), 3, 14)
    b = synth.normal_bf16((K, N), 3, 15)
    got = _gemm(dev, a, b)                    # variant 0: split-K with allocator scratch
    ref = oracle.gemm_bf16(a, b)
    _check(got, ref, K)
    unsplit = _gemm(dev, a, b, variant=4)
    gf, uf = synth.from_bf16(got), synth.from_bf16(unsplit)
    assert np.abs(gf - uf).max() <= 2 ** -7 * np.abs(uf).max()
    assert np.array_equal(got, _gemm(dev, a, b))
    # the same through a builtin Program with an explicit workspace buffer
    ws = lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)
    bc, bw = dev.buffer(M * N * 2), dev.buffer(ws)
    prog = morok_amd.Program.builtin("gemm_bf16", [M, N, K, 1, ws], dev.device_id)
    assert prog.name.endswith("_splitk")
    prog.execute([bc, ba, bb, bw])
    assert np.array_equal(bc.copyout(np.uint16, nbytes=M * N * 2).reshape(M, N), got)


def test_gemm_split_k_not_used_for_large_shapes():
    from morok_amd._ffi import lib

    for shape in [(4096, 4096, 4096), (512, 4096, 4096), (1024, 1024, 1024), (128, 256, 256), (8, 64, 128), (1024, 8192, 64)]:
        assert lib.mrk_hip_gemm_bf16_workspace_bytes(*shape, 1) == 0, shape


# (2148, 4096, 64) and (2148, 4104, 72) are large enough for the 256-row tile and end in a tile
# whose lower two waves lie entirely below row M.
@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 4096), (300, 264, 200), (128, 4096, 136), (1000, 520, 72), (257, 8, 8),
                                   (2148, 4096, 64), (2148, 4104, 72)])
def test_gemm_residual_epilogue(dev, oracle, shape):
    """c = a b + r with r added in the product kernel's epilogue: the bits of the plain
    product followed by an f32 add and one more rounding (the oracle's product, then numpy),
    for full, ragged and tiny tiles; memory behind c stays untouched and r is not read past
    its end (NaN patterns there would surface)."""
    M, N, K = shape
    a = synth.normal_bf16((M, K), 7, 41)
    b = synth.normal_bf16((K, N), 7, 42)
    r = synth.normal_bf16((M, N), 7, 43)
    nan = np.uint16(0x7FC0)
    rbig = np.full(M * N + 2048, nan, np.uint16)
    rbig[:M * N] = r.ravel()
    ba, bb, br = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (a, b, rbig))
    bc = morok_amd.Buffer.from_numpy(np.full(M * N + 2048, nan, np.uint16), dev.device_id)
    ops.gemm_bf16_residual(ba, bb, br, bc, M, N, K, dev.device_id)
    got = bc.copyout(np.uint16, (M * N + 2048,))
    assert np.all(got[M * N:] == nan)
    prod = oracle.gemm_bf16(a, b)
    want = synth.to_bf16(synth.from_bf16(prod) + synth.from_bf16(r))
    plain = dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, plain, M, N, K, dev.device_id)
    fused_from_plain = synth.to_bf16(synth.from_bf16(plain.copyout(np.uint16, (M, N))) + synth.from_bf16(r))
    assert np.array_equal(got[:M * N].reshape(M, N), fused_from_plain)
    gf, wf = synth.from_bf16(got[:M * N].reshape(M, N)), synth.from_bf16(want)
    assert np.abs(gf - wf).max() <= 2e-2 * np.abs(wf).max()


@pytest.mark.parametrize("shape", [(4, 1024, 4096), (1, 4096, 4096), (16, 12288, 512), (40, 4096, 2048), (100, 264, 4104), (200, 520, 8192)])
def test_gemm_residual_and_bias_where_the_product_is_spread_along_k(dev, shape):
    """Few output tiles against a long K, either layout of the weight: the product runs as the plain one does (split-K
    over the tiles, or the streaming kernels for a handful of rows) and the addend joins where the result is written,
    with the bits of the product followed by the elementwise add.  A matrix of the result's shape and a bias row."""
    M, N, K = shape
    a, b = synth.normal_bf16((M, K), 3, 50), synth.normal_bf16((K, N), 3, 51)
    r, bias = synth.normal_bf16((M, N), 3, 52), synth.normal_bf16((N,), 3, 53)
    ba, bb, br, bbias = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (a, b, r, bias))
    bbt = morok_amd.Buffer.from_numpy(np.ascontiguousarray(b.T), dev.device_id)
    plain, plain_nt = dev.buffer(M * N * 2), dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, plain, M, N, K, dev.device_id)
    ops.gemm_bf16_nt(ba, bbt, plain_nt, M, N, K, dev.device_id)
    p_kn, p_nt = synth.from_bf16(plain.copyout(np.uint16, (M, N))), synth.from_bf16(plain_nt.copyout(np.uint16, (M, N)))
    bc = morok_amd.Buffer.from_numpy(np.full(M * N + 2048, 0x7FC0, np.uint16), dev.device_id)
    ops.gemm_bf16_residual(ba, bb, br, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == 0x7FC0)
    assert np.array_equal(out[: M * N].reshape(M, N), synth.to_bf16(p_kn + synth.from_bf16(r)))
    ops.linear_bf16(ba, bbt, bbias, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    assert np.all(out[M * N:] == 0x7FC0)
    assert np.array_equal(out[: M * N].reshape(M, N), synth.to_bf16(p_nt + synth.from_bf16(bias)[None, :]))
    # as plan items with the plan's scratch, the other two combinations
    ws = morok_amd._ffi.lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    scratch = dev.buffer(max(ws, 16))
    params, bufs = ([M, N, K, 1, ws], [scratch]) if ws else ([M, N, K], [])
    morok_amd.Program.builtin("gemm_bf16_bias", params, dev.device_id).execute([bc, ba, bb, bbias] + bufs)
    assert np.array_equal(bc.copyout(np.uint16)[: M * N].reshape(M, N), synth.to_bf16(p_kn + synth.from_bf16(bias)[None, :]))
    if M <= 64:
        morok_amd.Program.builtin("gemm_bf16_nt_residual", [M, N, K], dev.device_id).execute([bc, ba, bbt, br])
        assert np.array_equal(bc.copyout(np.uint16)[: M * N].reshape(M, N), synth.to_bf16(p_nt + synth.from_bf16(r)))


def test_gemm_residual_refusals(dev):
    a = dev.buffer(4 * 4096 * 2)
    b = dev.buffer(4096 * 1024 * 2)
    c = dev.buffer(4 * 1024 * 2)
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_residual(a, b, c, c, 4, 1020, 64, dev.device_id)     # N not a multiple of 8
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_residual(a, b, c, c, 4, 1024, 60, dev.device_id)     # K not a multiple of 8


# ---------------------------------------------------------------- gated epilogue (SwiGLU)
@pytest.mark.parametrize("shape", [(256, 128, 64), (512, 1024, 256), (300, 1000, 192), (37, 136, 72), (1024, 11008 // 8, 512)])
def test_gemm_swiglu_epilogue_parity(dev, oracle, shape):
    """c = silu(a @ Wg) * (a @ Wu) with [Wg | Wu] stored side by side, the gate applied in the product
    kernel's epilogue: against the oracle's three stages (two bf16 products rounded to bf16, then
    orc_silu_mul_bf16) at the bf16 GEMM tolerance, and against the unfused GPU sequence (two
    products + the generated elementwise kernel), from which it may differ by the rounding of the
    fast reciprocal only: one bf16 ulp on a small fraction of the elements."""
    from morok_amd import tensor as T, uop

    M, F, K = shape
    a = synth.normal_bf16((M, K), 11, 0)
    w = synth.to_bf16(synth.normal((K, 2 * F), 11, 1, sigma=1.0 / np.sqrt(K)))
    ba, bw = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(w, dev.device_id)
    # NaNs right behind the result: the masked edge stores must not reach them
    out = dev.buffer(M * F * 2 + 256)
    out.copyin(np.full(M * F + 128, 0x7FC0, np.uint16))
    ops.gemm_bf16_swiglu(ba, bw, out, M, F, K, dev.device_id)
    raw = out.copyout(np.uint16, nbytes=M * F * 2 + 256)
    got, guard = raw[: M * F].reshape(M, F), raw[M * F:]
    assert np.all(guard == 0x7FC0)
    gate, up = oracle.gemm_bf16(a, np.ascontiguousarray(w[:, :F])), oracle.gemm_bf16(a, np.ascontiguousarray(w[:, F:]))
    ref = synth.from_bf16(oracle.silu_mul_bf16(gate, up))
    gf = synth.from_bf16(got)
    assert np.all(np.isfinite(gf))
    assert np.abs(gf - ref).max() <= 2e-2 * np.abs(ref).max()
    # the unfused path on the GPU
    T.set_fusion(True)
    ta, tw = T.Tensor.from_numpy(a, uop.BF16), T.Tensor.from_numpy(w, uop.BF16)
    g, u = ta.matmul(tw.try_shrink([(0, K), (0, F)]).contiguous()), ta.matmul(tw.try_shrink([(0, K), (F, 2 * F)]).contiguous())
    unfused = g.silu().try_mul(u).to_numpy()
    diff = got.astype(np.int32) - unfused.astype(np.int32)
    assert np.abs(diff).max() <= 1 and np.count_nonzero(diff) <= 0.02 * diff.size
    # and through the lazy graph: the scheduler picks the fused kernel for the packed product
    gu = ta.matmul(tw)
    fused = gu.try_shrink([(0, M), (0, F)]).silu().try_mul(gu.try_shrink([(0, M), (F, 2 * F)]))
    assert np.array_equal(fused.to_numpy(), got)
    assert [k for k in fused.kernels() if k.startswith("gemm_bf16_swiglu")], fused.kernels()


# ---------------------------------------------------------------- second operand stored [N, K]
# (a Linear layer's weight, tensor/src/nn/linear.rs:9-14: y = x @ weight.T + bias)
@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 256), (300, 520, 128), (1024, 1024, 1024), (1000, 776, 320),
                                   (100, 264, 200), (256, 256, 72), (129, 8, 72), (2048, 512, 136), (137, 4096, 64)])
def test_gemm_transposed_second_operand(dev, oracle, shape):
    """a @ bt.T with bt [N, K] read in place: the same products in the same order as the
    [K, N] form, so the same bits, on full, ragged-M/N and ragged-K shapes and with either tile
    size; NaNs right behind a, bt and c show that no edge reads or writes past them."""
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 20)
    b = synth.normal_bf16((K, N), 3, 21)
    bt = np.ascontiguousarray(b.T)
    nan = np.full(8192, 0x7FC0, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.reshape(-1), nan]), dev.device_id)
    bbt = morok_amd.Buffer.from_numpy(np.concatenate([bt.reshape(-1), nan]), dev.device_id)
    bc = dev.buffer(M * N * 2 + 4096)
    bc.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.gemm_bf16_nt(ba, bbt, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    got = out[: M * N].reshape(M, N)
    assert np.all(out[M * N:] == 0x7FC0)
    _check(got, oracle.gemm_bf16(a, b), K)
    assert np.array_equal(got, _gemm(dev, a, b, variant=3))
    # and as a plan item
    bc2 = dev.buffer(M * N * 2)
    morok_amd.Program.builtin("gemm_bf16_nt", [M, N, K], dev.device_id).execute([bc2, ba, bbt])
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)


def test_gemm_transposed_second_operand_refusals(dev):
    a, b, c = dev.buffer(72 * 4096 * 2), dev.buffer(4096 * 1024 * 2), dev.buffer(72 * 1024 * 2)
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_nt(a, b, c, 32, 1024, 4092, dev.device_id)  # K not a multiple of 8
    with pytest.raises(morok_amd.MorokHipError):
        ops.gemm_bf16_nt(a, b, c, 72, 1020, 64, dev.device_id)    # N not a multiple of 8 with more than 64 rows


@pytest.mark.parametrize("shape", [(72, 1024, 4096), (96, 4096, 4096), (65, 520, 2048), (100, 264, 4104), (80, 4096, 8192), (128, 512, 8192)])
def test_gemm_transposed_second_operand_split_k(dev, oracle, shape):
    """Few output tiles against a long K with the weight stored [N, K] and more than 64 rows: the K loop is spread over the
    chip as for the [K, N] form (same K ranges, same order inside a range: the same bits), through the
    ABI (which brings the scratch itself) and as a plan item with a scratch buffer."""
    M, N, K = shape
    ws = morok_amd._ffi.lib.mrk_hip_gemm_bf16_workspace_bytes(M, N, K, 1)
    assert ws > 0
    a = synth.normal_bf16((M, K), 3, 30)
    b = synth.normal_bf16((K, N), 3, 31)
    bt = np.ascontiguousarray(b.T)
    nan = np.full(8192, 0x7FC0, np.uint16)
    ba = morok_amd.Buffer.from_numpy(np.concatenate([a.reshape(-1), nan]), dev.device_id)
    bbt = morok_amd.Buffer.from_numpy(np.concatenate([bt.reshape(-1), nan]), dev.device_id)
    bc = dev.buffer(M * N * 2 + 4096)
    bc.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.gemm_bf16_nt(ba, bbt, bc, M, N, K, dev.device_id)
    out = bc.copyout(np.uint16)
    got = out[: M * N].reshape(M, N)
    assert np.all(out[M * N:] == 0x7FC0)
    _check(got, oracle.gemm_bf16(a, b), K)
    assert np.array_equal(got, _gemm(dev, a, b))
    bc2, scratch = dev.buffer(M * N * 2), dev.buffer(ws)
    morok_amd.Program.builtin("gemm_bf16_nt", [M, N, K, 1, ws], dev.device_id).execute([bc2, ba, bbt, scratch])
    assert np.array_equal(bc2.copyout(np.uint16, (M, N)), got)


LINEAR_SHAPES = [(256, 256, 64), (512, 768, 256), (300, 520, 128), (1000, 776, 320), (2048, 512, 136),   # tiled kernels
                 (1, 4096, 4096), (2, 1020, 64), (5, 37, 520), (16, 4096, 1024), (33, 515, 264), (64, 12288, 512)]  # streamed


@pytest.mark.parametrize("shape", LINEAR_SHAPES)
def test_linear_forward_with_bias(dev, oracle, shape):
    """y = x @ w.T + bias with w [out, in] and bias [out] as nn::Linear holds them (tensor/src/nn/linear.rs:9-14,
    39-41), the bias added in the product kernel's epilogue: the bits of the product (same kernel family, no bias)
    followed by the elementwise add in bf16, within the GEMM tolerance of the oracle; NaNs right behind every
    operand and the result; bias = None is the plain product."""
    M, N, K = shape
    x = synth.normal_bf16((M, K), 3, 40)
    w = synth.normal_bf16((N, K), 3, 41)
    bias = synth.normal_bf16((N,), 3, 42)
    nan = np.full(8192, 0x7FC0, np.uint16)
    bx = morok_amd.Buffer.from_numpy(np.concatenate([x.reshape(-1), nan]), dev.device_id)
    bw = morok_amd.Buffer.from_numpy(np.concatenate([w.reshape(-1), nan]), dev.device_id)
    bb = morok_amd.Buffer.from_numpy(np.concatenate([bias, nan]), dev.device_id)
    by = dev.buffer(M * N * 2 + 4096)
    by.copyin(np.full(M * N + 2048, 0x7FC0, np.uint16))
    ops.linear_bf16(bx, bw, bb, by, M, N, K, dev.device_id)
    out = by.copyout(np.uint16)
    got = out[: M * N].reshape(M, N)
    assert np.all(out[M * N:] == 0x7FC0)
    bp = dev.buffer(M * N * 2)
    ops.linear_bf16(bx, bw, None, bp, M, N, K, dev.device_id)
    prod = bp.copyout(np.uint16, (M, N))
    bp2 = dev.buffer(M * N * 2)
    ops.gemm_bf16_nt(bx, bw, bp2, M, N, K, dev.device_id)
    assert np.array_equal(prod, bp2.copyout(np.uint16, (M, N)))
    want = synth.to_bf16(synth.from_bf16(prod) + synth.from_bf16(bias)[None, :])
    assert np.array_equal(got, want)
    ref = synth.from_bf16(oracle.gemm_bf16(x, np.ascontiguousarray(w.T))) + synth.from_bf16(bias)[None, :]
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # as plan items, for either layout of the weight
    by2 = dev.buffer(M * N * 2)
    morok_amd.Program.builtin("gemm_bf16_nt_bias", [M, N, K], dev.device_id).execute([by2, bx, bw, bb])
    assert np.array_equal(by2.copyout(np.uint16, (M, N)), got)
    if N % 8 == 0:
        bwt = morok_amd.Buffer.from_numpy(np.ascontiguousarray(w.T), dev.device_id)
        morok_amd.Program.builtin("gemm_bf16_bias", [M, N, K], dev.device_id).execute([by2, bx, bwt, bb])
        kn = synth.from_bf16(by2.copyout(np.uint16, (M, N)))
        if M > 64:
            assert np.array_equal(by2.copyout(np.uint16, (M, N)), got)      # the tiled kernels: the same bits in either layout
        else:
            assert np.abs(kn - ref).max() <= 2e-2 * np.abs(ref).max()


def test_linear_forward_with_bias_few_tiles_and_refusals(dev, oracle):
    """More than 64 rows with few output tiles against a long K: the product is spread along K as the plain one is and
    the bias is added where the partial results are summed; K not a multiple of 8 is refused."""
    M, N, K = 100, 264, 4104
    x, w, bias = synth.normal_bf16((M, K), 3, 43), synth.normal_bf16((N, K), 3, 44), synth.normal_bf16((N,), 3, 45)
    bx, bw, bb = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (x, w, bias))
    by, bp = dev.buffer(M * N * 2), dev.buffer(M * N * 2)
    ops.linear_bf16(bx, bw, bb, by, M, N, K, dev.device_id)
    ops.gemm_bf16_nt(bx, bw, bp, M, N, K, dev.device_id)
    want = synth.to_bf16(synth.from_bf16(bp.copyout(np.uint16, (M, N))) + synth.from_bf16(bias)[None, :])
    assert np.array_equal(by.copyout(np.uint16, (M, N)), want)
    ref = synth.from_bf16(oracle.gemm_bf16(x, np.ascontiguousarray(w.T))) + synth.from_bf16(bias)[None, :]
    assert np.abs(synth.from_bf16(by.copyout(np.uint16, (M, N))) - ref).max() <= 2e-2 * np.abs(ref).max()
    with pytest.raises(morok_amd.MorokHipError):
        ops.linear_bf16(bx, bw, bb, by, M, N, 4100, dev.device_id)
    with pytest.raises(morok_amd.MorokHipError):
        ops.linear_bf16(bx, bw, bb, by, M, 260, K, dev.device_id)       # more than 64 rows and N not a multiple of 8


@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 1024), (300, 264, 200), (1000, 520, 72)])
def test_gemm_transposed_second_operand_epilogues(dev, shape):
    """The residual and the gated epilogue over a [N, K] ([2F, K]) second operand, as plan items:
    the bits of the same epilogues over the [K, N] form."""
    M, N, K = shape
    a = synth.normal_bf16((M, K), 7, 51)
    b = synth.normal_bf16((K, N), 7, 52)
    r = synth.normal_bf16((M, N), 7, 53)
    ba, bb, bbt, br = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (a, b, np.ascontiguousarray(b.T), r))
    c0, c1 = dev.buffer(M * N * 2), dev.buffer(M * N * 2)
    morok_amd.Program.builtin("gemm_bf16_residual", [M, N, K], dev.device_id).execute([c0, ba, bb, br])
    morok_amd.Program.builtin("gemm_bf16_nt_residual", [M, N, K], dev.device_id).execute([c1, ba, bbt, br])
    assert np.array_equal(c0.copyout(np.uint16, (M, N)), c1.copyout(np.uint16, (M, N)))
    F = N // 2
    if F % 8 == 0:
        w = synth.to_bf16(synth.normal((K, 2 * F), 11, 1, sigma=1.0 / np.sqrt(K)))
        bw, bwt = morok_amd.Buffer.from_numpy(w, dev.device_id), morok_amd.Buffer.from_numpy(np.ascontiguousarray(w.T), dev.device_id)
        g0, g1 = dev.buffer(M * F * 2), dev.buffer(M * F * 2)
        morok_amd.Program.builtin("gemm_bf16_swiglu", [M, F, K], dev.device_id).execute([g0, ba, bw])
        morok_amd.Program.builtin("gemm_bf16_nt_swiglu", [M, F, K], dev.device_id).execute([g1, ba, bwt])
        assert np.array_equal(g0.copyout(np.uint16, (M, F)), g1.copyout(np.uint16, (M, F)))


@pytest.mark.parametrize("shape", [(256, 768, 128, 512, 64), (512, 1536, 256, 1024, 128), (300, 512, 192, 512, 100), (1000, 1288, 320, 768, 77),
                                   (256, 512, 64, 256, 256), (256, 512, 128, 512, 32)])
def test_gemm_rotary_epilogue(dev, oracle, shape):
    """The packed projection with the rotary embedding of its first `split` columns (heads of 128) in
    the product's epilogue: against the oracle's product followed by its rotary stage on the
    bf16-rounded product (f32 arithmetic, one rounding) and against the plain product for the
    unrotated rest; rows past a multiple of 256, a rest that is not a multiple of 256 columns and
    positions that wrap (row % seq) included; NaNs behind both results show nothing is written past them."""
    M, N, K, split, seq = shape
    a = synth.normal_bf16((M, K), 3, 30)
    b = synth.normal_bf16((K, N), 3, 31)
    ang = synth.uniform((seq, 64), 3, 32) * np.float32(3.0)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)
    bcos, bsin = morok_amd.Buffer.from_numpy(cos, dev.device_id), morok_amd.Buffer.from_numpy(sin, dev.device_id)
    rest = N - split
    brot = morok_amd.Buffer.from_numpy(np.full(M * split + 2048, 0x7FC0, np.uint16), dev.device_id)
    brest = morok_amd.Buffer.from_numpy(np.full(M * rest + 2048, 0x7FC0, np.uint16), dev.device_id)
    ops.gemm_bf16_rope(ba, bb, bcos, bsin, brot, brest, M, N, K, split, seq, dev.device_id)
    rot_all, rest_all = brot.copyout(np.uint16), brest.copyout(np.uint16)
    assert np.all(rot_all[M * split:] == 0x7FC0) and np.all(rest_all[M * rest:] == 0x7FC0)
    got_rot, got_rest = rot_all[: M * split].reshape(M, split), rest_all[: M * rest].reshape(M, rest)
    plain = _gemm(dev, a, b)
    assert np.array_equal(got_rest, plain[:, split:])                        # the unrotated columns: the plain product's bits
    heads = split // 128
    x = synth.from_bf16(plain[:, :split]).reshape(M, heads, 128)             # the bf16-rounded product, as the separate kernel reads it
    pos = np.arange(M) % seq
    want = oracle.rope_f32(x, cos[pos][:, None, :], sin[pos][:, None, :], False).reshape(M, split)
    gf = synth.from_bf16(got_rot)
    assert np.all(np.isfinite(gf))
    # the same arithmetic up to the contraction of a multiply-add: within one bf16 rounding of the f32 result
    assert np.all(np.abs(gf - want) <= np.abs(want) * 2.0 ** -7 + 1e-6 * np.abs(x).max())
    ref_prod = synth.from_bf16(oracle.gemm_bf16(a, b))[:, :split].reshape(M, heads, 128)
    ref = oracle.rope_f32(ref_prod, cos[pos][:, None, :], sin[pos][:, None, :], False).reshape(M, split)
    assert np.abs(gf - ref).max() <= 2e-2 * np.abs(ref).max()
    # as a plan item
    brot2, brest2 = dev.buffer(M * split * 2), dev.buffer(max(M * rest * 2, 2))
    morok_amd.Program.builtin("gemm_bf16_rope", [M, N, K, split, seq], dev.device_id).execute([brot2, ba, bb, brest2, bcos, bsin])
    assert np.array_equal(brot2.copyout(np.uint16, (M, split)), got_rot)
    # with the weight stored [N, K] (a Linear layer's): the same products in the same order, so the same bits
    bbt = morok_amd.Buffer.from_numpy(np.ascontiguousarray(b.T), dev.device_id)
    brot3 = morok_amd.Buffer.from_numpy(np.full(M * split + 2048, 0x7FC0, np.uint16), dev.device_id)
    brest3 = morok_amd.Buffer.from_numpy(np.full(M * rest + 2048, 0x7FC0, np.uint16), dev.device_id)
    morok_amd.Program.builtin("gemm_bf16_nt_rope", [M, N, K, split, seq], dev.device_id).execute([brot3, ba, bbt, brest3, bcos, bsin])
    assert np.array_equal(brot3.copyout(np.uint16), rot_all) and np.array_equal(brest3.copyout(np.uint16), rest_all)


def test_gemm_rotary_epilogue_refusals(dev):
    b = dev.buffer(1 << 20).ensure_allocated()
    for (m, n, k, split, seq) in [(64, 512, 72, 256, 8), (64, 512, 64, 128, 8), (64, 512, 64, 768, 8), (64, 508, 64, 256, 8), (64, 512, 64, 256, 0)]:
        with pytest.raises(morok_amd.MorokHipError):
            ops.gemm_bf16_rope(b, b, b, b, b, b, m, n, k, split, seq, dev.device_id)
