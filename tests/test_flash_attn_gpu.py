"""Parity of the fused flash-attention forward with the CPU oracle's SDPA (policy 0: f32
scores and softmax statistics, P rounded to bf16 before P.V, bf16 output) on identical
seeded inputs.  Tolerance from the north star: <= 2e-2 max relative error for bf16
attention with fp32 accumulate, measured as max|gpu - ref| / max|ref|."""
import numpy as np
import pytest

import morok_amd
from morok_amd import MorokHipError, ops, synth

pytestmark = pytest.mark.gpu
D = 128


def _attn(dev, q, k, v, scale, causal, via_program=False):
    B, H, Sq, _ = q.shape
    Sk = k.shape[2]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    bo = dev.buffer(q.nbytes)
    if via_program:
        bits = int(np.float32(scale).view(np.uint32))
        prog = morok_amd.Program.builtin("flash_fwd_bf16", [B * H, Sq, Sk, D, int(causal), bits], dev.device_id)
        prog.execute([bo, bq, bk, bv])
    else:
        ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, Sq, Sk, D, scale, causal, dev.device_id)
    return bo.copyout(np.uint16, q.shape)


def _inputs(B, H, Sq, Sk, seed=4):
    return (synth.normal_bf16((B, H, Sq, D), seed, 0), synth.normal_bf16((B, H, Sk, D), seed, 1),
            synth.normal_bf16((B, H, Sk, D), seed, 2))


def _check(o, ref):
    of, rf = synth.from_bf16(o), synth.from_bf16(ref)
    assert np.all(np.isfinite(of))
    err = np.abs(of - rf).max() / np.abs(rf).max()
    assert err <= 2e-2, err
    # in practice the two agree to a few bf16 ulps of the row scale
    assert err <= 8e-3, err


SCALE = 1.0 / np.sqrt(D)


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (1, 2, 64, 64), (2, 3, 80, 80), (1, 1, 128, 128), (1, 2, 129, 129),
                                   (1, 1, 300, 300), (2, 2, 512, 512), (1, 3, 33, 257), (1, 1, 257, 33)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_parity_shapes(dev, oracle, shape, causal):
    B, H, Sq, Sk = shape
    q, k, v = _inputs(B, H, Sq, Sk)
    _check(_attn(dev, q, k, v, SCALE, causal), oracle.sdpa_bf16(q, k, v, SCALE, causal=causal))


def test_flash_special_cases(dev):
    B, H, S = 2, 2, 256
    q, k, v = _inputs(B, H, S, S, seed=14)
    o = _attn(dev, q, k, v, SCALE, True)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])  # first causal row sees key 0 only (reference test row0 == V[0])
    # uniform K: every visible key scores the same -> causal running mean of V
    k1 = np.broadcast_to(k[:, :, :1], k.shape).copy()
    o = synth.from_bf16(_attn(dev, q, k1, v, SCALE, True))
    run = np.cumsum(synth.from_bf16(v).astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert np.abs(o - run).max() < 2e-2
    # one-hot attention: huge score on key (i // 2) -> output row i == V[i // 2] exactly
    qh = np.zeros((1, 1, S, D), np.float32)
    kh = np.zeros((1, 1, S, D), np.float32)
    for i in range(S):
        kh[0, 0, i, i % D] = 16.0 * (1 + i // D)
    for i in range(S):
        t = i // 2
        qh[0, 0, i, t % D] = 16.0 * (1 + t // D)
    # make keys distinguishable across the i // D bands: matching band gives the largest product only
    # when magnitudes match, so use distinct one-hot columns within a band and bands of 128 keys <= S
    S2 = 128
    o = _attn(dev, synth.to_bf16(qh[:, :, :S2]), synth.to_bf16(kh[:, :, :S2]), v[:1, :1, :S2], 1.0, True)
    want = v[:1, :1, np.arange(S2) // 2]
    assert np.array_equal(o, want)


@pytest.mark.parametrize("trend", ["rising", "falling", "spiky"])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_score_ranges(dev, oracle, trend, causal):
    """Scores far outside the comfortable range: maxima that keep growing along the keys force
    a rescale of the accumulators at every tile, falling ones none after the first, isolated
    spikes of +-200 exercise the reference-point logic in both directions."""
    B, H, S = 1, 2, 512
    q, k, v = _inputs(B, H, S, S, seed=21)
    qf, kf = synth.from_bf16(q).copy(), synth.from_bf16(k).copy()
    qf[..., 0] = 1.0
    j = np.arange(S, dtype=np.float32)
    if trend == "rising":
        kf[..., 0] = 0.4 * j              # +25.6 per 64-key tile
    elif trend == "falling":
        kf[..., 0] = -0.4 * j
    else:
        kf[..., 0] = 0.0
        kf[:, :, 70::97, 0] = 200.0
        kf[:, :, 33::131, 0] = -200.0
    q2, k2 = synth.to_bf16(qf), synth.to_bf16(kf)
    _check(_attn(dev, q2, k2, v, 1.0, causal), oracle.sdpa_bf16(q2, k2, v, 1.0, causal=causal))


@pytest.mark.parametrize("shape", [(1, 2, 100, 100), (1, 1, 129, 257), (2, 1, 64, 33), (1, 1, 1, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_does_not_touch_neighbours(dev, oracle, shape, causal):
    """Ragged last tiles: NaNs right behind Q, K and V in their allocations do not reach O, and
    nothing is written behind O."""
    B, H, Sq, Sk = shape
    q, k, v = _inputs(B, H, Sq, Sk, seed=23)
    nan = np.full(4096, 0x7FC0, np.uint16)
    bq, bk, bv = (morok_amd.Buffer.from_numpy(np.concatenate([t.reshape(-1), nan]), dev.device_id) for t in (q, k, v))
    bo = morok_amd.Buffer.from_numpy(np.full(q.size + 4096, 0x7FC0, np.uint16), dev.device_id)
    ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, Sq, Sk, D, SCALE, causal, dev.device_id)
    out = bo.copyout(np.uint16)
    _check(out[: q.size].reshape(q.shape), oracle.sdpa_bf16(q, k, v, SCALE, causal=causal))
    assert np.all(out[q.size:] == 0x7FC0)


def test_flash_program_path_and_errors(dev, oracle):
    q, k, v = _inputs(1, 2, 192, 192, seed=24)
    _check(_attn(dev, q, k, v, SCALE, True, via_program=True), oracle.sdpa_bf16(q, k, v, SCALE, causal=True))
    with pytest.raises(MorokHipError) as e:
        ops.flash_attn_fwd_bf16(1, 1, 1, 1, 1, 1, 16, 16, 96, SCALE, True, dev.device_id)
    assert e.value.code == 11 and "head_dim" in e.value.message
    with pytest.raises(MorokHipError):
        ops.flash_attn_fwd_bf16(1, 1, 1, 1, 1, 1, 16, 0, 128, SCALE, True, dev.device_id)
    with pytest.raises(MorokHipError):
        ops.flash_attn_fwd_bf16(1, 1, 1, 1, 1, 1, 16, 16, 128, -1.0, True, dev.device_id)
    ops.flash_attn_fwd_bf16(0, 0, 0, 0, 0, 4, 16, 16, 128, SCALE, True, dev.device_id)  # empty batch: no-op


def test_flash_config_slice_s4096(dev, oracle):
    # two heads of the benchmark shape (seq 4096, head_dim 128, causal, scale 1/sqrt(128))
    q, k, v = _inputs(1, 2, 4096, 4096)
    _check(_attn(dev, q, k, v, SCALE, True), oracle.sdpa_bf16(q, k, v, SCALE, causal=True))


def test_flash_full_size_properties(dev, oracle):
    # configs[3] full size: bf16 [8, 32, 4096, 128]; size-independent properties + sampled heads
    B, H, S = 8, 32, 4096
    q, k, v = _inputs(B, H, S, S)
    o = _attn(dev, q, k, v, SCALE, True)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])
    # linearity in V: scaling V by 2 is exact in bf16 and f32 -> bitwise doubled output
    v2 = synth.to_bf16(synth.from_bf16(v) * 2)
    o2 = _attn(dev, q, k, v2, SCALE, True)
    assert np.array_equal(synth.from_bf16(o2), synth.from_bf16(o) * 2)
    # convex combination: every output lies inside the running min/max envelope of V
    vf = synth.from_bf16(v[3, 5])
    of = synth.from_bf16(o[3, 5])
    hi = np.maximum.accumulate(vf, axis=0)
    lo = np.minimum.accumulate(vf, axis=0)
    assert np.all(of <= hi + 2e-2) and np.all(of >= lo - 2e-2)
    for b, h in ((0, 0), (7, 31)):
        ref = oracle.sdpa_bf16(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], SCALE, causal=True)
        _check(o[b:b + 1, h:h + 1], ref)


@pytest.mark.parametrize("seed", range(16))
def test_flash_random_shapes(dev, oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    Sq, Sk = int(rng.integers(1, 520)), int(rng.integers(1, 520))
    causal = bool(seed & 1)
    scale = float(rng.choice([SCALE, 0.05, 0.2]))
    q, k, v = _inputs(B, H, Sq, Sk, seed=40 + seed)
    _check(_attn(dev, q, k, v, scale, causal), oracle.sdpa_bf16(q, k, v, scale, causal=causal))


# ---------------------------------------------------------------- operands given as views
def _strided(dev, bufs, offsets, strides, B, H, Sq, Sk, causal, o_init=None, via_program=False):
    """Runs the strided entry point on host arrays `bufs` = (q, k, v, o-shaped uint16 arrays of
    whatever layout) and returns the output buffer's contents in its own layout."""
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in bufs[:3])
    o_host = bufs[3] if o_init is None else o_init
    bo = morok_amd.Buffer.from_numpy(o_host, dev.device_id)
    if via_program:
        bits = int(np.float32(SCALE).view(np.uint32))
        prog = morok_amd.Program.builtin("flash_fwd_bf16_strided",
                                         [B, H, Sq, Sk, D, int(causal), bits, *offsets, *strides], dev.device_id)
        prog.execute([bo, bq, bk, bv])
    else:
        ops.flash_attn_fwd_bf16_strided(bq, bk, bv, bo, B, H, Sq, Sk, D, SCALE, strides, offsets, causal, dev.device_id)
    return bo.copyout(np.uint16, o_host.shape)


@pytest.mark.parametrize("shape", [(2, 3, 200, 200), (1, 4, 129, 257), (2, 2, 384, 384)])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("via_program", [False, True])
def test_flash_over_seq_major_views(dev, oracle, shape, causal, via_program):
    """All four operands as [B, S, H, D] activations (what a projection writes), the kernel
    told so through strides: the same bits as the kernel over [B, H, S, D] copies, and the
    oracle's values."""
    B, H, Sq, Sk = shape
    q, k, v = _inputs(B, H, Sq, Sk, seed=31)
    qs, ks, vs = (np.ascontiguousarray(t.transpose(0, 2, 1, 3)) for t in (q, k, v))
    strides = [Sq * H * D, D, H * D, Sk * H * D, D, H * D, Sk * H * D, D, H * D, Sq * H * D, D, H * D]
    o = _strided(dev, (qs, ks, vs, np.zeros_like(qs)), [0, 0, 0, 0], strides, B, H, Sq, Sk, causal, via_program=via_program)
    o = o.transpose(0, 2, 1, 3)
    assert np.array_equal(o, _attn(dev, q, k, v, SCALE, causal))
    _check(o, oracle.sdpa_bf16(q, k, v, SCALE, causal=causal))


def test_flash_over_a_packed_qkv_product(dev):
    """q, k and v as column slices of one [B*S, 3*H*D] matrix (a fused QKV projection), the
    output as a column slice of a wider matrix whose other columns must stay as they were."""
    B, H, S = 2, 4, 320
    q, k, v = _inputs(B, H, S, S, seed=32)
    hid = H * D
    packed = np.zeros((B, S, 3 * hid), np.uint16)
    for i, t in enumerate((q, k, v)):
        packed[:, :, i * hid:(i + 1) * hid] = t.transpose(0, 2, 1, 3).reshape(B, S, hid)
    wide = np.full((B, S, hid + 64), 0x7FC0, np.uint16)  # bf16 NaN pattern: writes outside the view would show
    st_in = [S * 3 * hid, D, 3 * hid]
    strides = st_in * 3 + [S * (hid + 64), D, hid + 64]
    o = _strided(dev, (packed, packed, packed, None), [0, hid, 2 * hid, 32], strides, B, H, S, S, True, o_init=wide)
    assert np.all(o[:, :, :32] == 0x7FC0) and np.all(o[:, :, 32 + hid:] == 0x7FC0)
    got = o[:, :, 32:32 + hid].reshape(B, S, H, D).transpose(0, 2, 1, 3)
    assert np.array_equal(got, _attn(dev, q, k, v, SCALE, True))


def test_flash_shared_keys_through_zero_strides(dev, oracle):
    """One set of keys and values for every head (head stride 0) and for every batch (batch
    stride 0): the same as the kernel over broadcast copies."""
    B, H, Sq, Sk = 2, 3, 150, 260
    q, _, _ = _inputs(B, H, Sq, Sk, seed=33)
    k1 = synth.normal_bf16((1, 1, Sk, D), 33, 1)
    v1 = synth.normal_bf16((1, 1, Sk, D), 33, 2)
    strides = [H * Sq * D, Sq * D, D, 0, 0, D, 0, 0, D, H * Sq * D, Sq * D, D]
    o = _strided(dev, (q, k1, v1, np.zeros_like(q)), [0, 0, 0, 0], strides, B, H, Sq, Sk, False)
    kb, vb = (np.ascontiguousarray(np.broadcast_to(t, (B, H, Sk, D))) for t in (k1, v1))
    assert np.array_equal(o, _attn(dev, q, kb, vb, SCALE, False))
    _check(o, oracle.sdpa_bf16(q, kb, vb, SCALE, causal=False))


def test_flash_dense_strides_take_the_plain_kernel(dev):
    B, H, S = 1, 2, 256
    q, k, v = _inputs(B, H, S, S, seed=34)
    strides = [H * S * D, S * D, D] * 4
    o = _strided(dev, (q, k, v, np.zeros_like(q)), [0, 0, 0, 0], strides, B, H, S, S, True)
    assert np.array_equal(o, _attn(dev, q, k, v, SCALE, True))


def test_flash_strided_refuses_what_it_cannot_address(dev):
    B, H, S = 1, 2, 64
    q, k, v = _inputs(B, H, S, S, seed=35)
    good = [H * S * D, S * D, D] * 4
    bufs = (q, k, v, np.zeros_like(q))
    for i, bad in ((2, D + 4), (1, S * D + 1), (11, 64), (10, 0)):  # unaligned row / head stride, overlapping output rows / heads
        st = list(good)
        st[i] = bad
        with pytest.raises((MorokHipError, ValueError)):
            _strided(dev, bufs, [0, 0, 0, 0], st, B, H, S, S, True)
    with pytest.raises((MorokHipError, ValueError)):  # unaligned offset
        _strided(dev, bufs, [4, 0, 0, 0], good, B, H, S, S, True)
    with pytest.raises(ValueError):  # the view reaches past the buffer
        _strided(dev, bufs, [0, 0, 0, 0], [H * S * D, S * D, 2 * D] + good[3:], B, H, S, S, True)


# ---------------------------------------------------------------- head dims 64 and 256
def _attn_d(dev, q, k, v, scale, causal, d):
    B, H, Sq, _ = q.shape
    Sk = k.shape[2]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    bo = dev.buffer(q.nbytes)
    ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, causal, dev.device_id)
    return bo.copyout(np.uint16, q.shape)


def _inputs_d(B, H, Sq, Sk, d, seed):
    return (synth.normal_bf16((B, H, Sq, d), seed, 0), synth.normal_bf16((B, H, Sk, d), seed, 1),
            synth.normal_bf16((B, H, Sk, d), seed, 2))


@pytest.mark.parametrize("d", [64, 256])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (1, 2, 64, 64), (2, 3, 80, 80), (1, 2, 129, 129), (1, 1, 300, 300),
                                   (2, 2, 512, 512), (1, 3, 33, 257), (1, 1, 257, 33), (1, 2, 1024, 1024)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_other_head_dims_parity_shapes(dev, oracle, shape, causal, d):
    """The head-dim-64 and head-dim-256 instantiations of the same kernel body (128-byte rows in
    LDS with their own K swizzle; 512-byte rows, one workgroup per CU, an exponential pair behind
    every second score MFMA): the same cases as head dim 128 against the oracle, scale 1/sqrt(d)."""
    B, H, Sq, Sk = shape
    q, k, v = _inputs_d(B, H, Sq, Sk, d, seed=61)
    sc = float(d) ** -0.5
    _check(_attn_d(dev, q, k, v, sc, causal, d), oracle.sdpa_bf16(q, k, v, sc, causal=causal))


@pytest.mark.parametrize("d", [64, 256])
def test_flash_other_head_dims_special_cases_and_bounds(dev, oracle, d):
    B, H, S = 2, 2, 256
    sc = float(d) ** -0.5
    q, k, v = _inputs_d(B, H, S, S, d, seed=62)
    o = _attn_d(dev, q, k, v, sc, True, d)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])   # first causal row sees key 0 only
    # every d column is used: a one-hot V picks single columns of P's row sums (all ones)
    rows = d + 6
    ones = synth.to_bf16(np.ones((1, 1, rows, d), np.float32))
    eye_rows = np.tile(np.eye(d, dtype=np.float32), (2, 1))[:rows]
    o = synth.from_bf16(_attn_d(dev, ones, ones, synth.to_bf16(eye_rows[None, None]), sc, False, d))
    want = eye_rows.sum(0) / float(rows)
    assert np.abs(o - want[None, None, None, :]).max() <= 2e-2 * want.max()
    # NaNs right behind every operand and the result (ragged last tiles)
    for Sq, Sk, causal in ((100, 100, True), (129, 257, False), (64, 33, True)):
        q, k, v = _inputs_d(1, 2, Sq, Sk, d, seed=63)
        nan = np.full(4096, 0x7FC0, np.uint16)
        bq, bk, bv = (morok_amd.Buffer.from_numpy(np.concatenate([t.reshape(-1), nan]), dev.device_id) for t in (q, k, v))
        bo = morok_amd.Buffer.from_numpy(np.full(q.size + 4096, 0x7FC0, np.uint16), dev.device_id)
        ops.flash_attn_fwd_bf16(bq, bk, bv, bo, 1, 2, Sq, Sk, d, sc, causal, dev.device_id)
        out = bo.copyout(np.uint16)
        _check(out[: q.size].reshape(q.shape), oracle.sdpa_bf16(q, k, v, sc, causal=causal))
        assert np.all(out[q.size:] == 0x7FC0)


@pytest.mark.parametrize("d", [64, 256])
def test_flash_other_head_dims_views_and_tensor_api(dev, oracle, d):
    """[B, S, H, d] activations through the strided entry point, and head dims 64 / 256 through
    Tensor::scaled_dot_product_attention (one fused kernel instead of the composed graph)."""
    from morok_amd import tensor as T, uop

    B, H, S = 2, 3, 200
    sc = float(d) ** -0.5
    q, k, v = _inputs_d(B, H, S, S, d, seed=64)
    qs, ks, vs = (np.ascontiguousarray(t.transpose(0, 2, 1, 3)) for t in (q, k, v))
    strides = [S * H * d, d, H * d] * 4
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (qs, ks, vs))
    bo = morok_amd.Buffer.from_numpy(np.zeros_like(qs), dev.device_id)
    ops.flash_attn_fwd_bf16_strided(bq, bk, bv, bo, B, H, S, S, d, sc, strides, [0, 0, 0, 0], True, dev.device_id)
    o = bo.copyout(np.uint16, qs.shape).transpose(0, 2, 1, 3)
    assert np.array_equal(o, _attn_d(dev, q, k, v, sc, True, d))
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16),
                                                                      T.Tensor.from_numpy(v, uop.BF16), is_causal=True)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16") and t.kernels()[0].endswith("_d%d" % d)
    assert np.array_equal(got, o)
    _check(got, oracle.sdpa_bf16(q, k, v, sc, causal=True))


@pytest.mark.parametrize("d", [64, 256])
@pytest.mark.parametrize("seed", range(8))
def test_flash_other_head_dims_random_shapes(dev, oracle, seed, d):
    rng = np.random.default_rng(5000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    Sq, Sk = int(rng.integers(1, 520)), int(rng.integers(1, 520))
    q, k, v = _inputs_d(B, H, Sq, Sk, d, seed=70 + seed)
    scale = float(rng.choice([0.125, 0.05, 0.2])) * (64.0 / d) ** 0.5
    _check(_attn_d(dev, q, k, v, scale, bool(seed & 1), d), oracle.sdpa_bf16(q, k, v, scale, causal=bool(seed & 1)))


@pytest.mark.parametrize("d,causal", [(96, True), (80, False), (40, True), (192, True), (8, False)])
def test_head_dims_without_an_instantiation_are_padded(dev, oracle, d, causal):
    """Tensor::scaled_dot_product_attention on a head dim with no fused instantiation: q, k, v are
    padded with zero columns to the next one that has (zero columns add exact zeros to the scores,
    the padded output columns are cut off), so the fused kernel runs and no [Sq, Sk] score matrix
    is materialised; the scale is that of the real head dim."""
    from morok_amd import tensor as T, uop

    B, H, S = 2, 2, 300
    q, k, v = _inputs_d(B, H, S, S, d, seed=81)
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16),
                                                                      T.Tensor.from_numpy(v, uop.BF16), is_causal=causal)
    got = t.to_numpy()
    names = t.kernels()
    assert sum(nm.startswith("flash_fwd_bf16") for nm in names) == 1 and not any(nm.startswith("r_") for nm in names), names
    assert got.shape == q.shape
    _check(got, oracle.sdpa_bf16(q, k, v, float(d) ** -0.5, causal=causal))


# ---------------------------------------------------------------- attn_mask and softcap inside the kernel
def _mask_for(kind, layout, B, H, Sq, Sk, seed):
    """(host array for the oracle, element strides per batch / head / row) of a mask broadcastable to
    [B, H, Sq, Sk]: Bool with ~60 % of the keys kept (key 0 always, so no row is empty) or additive bf16."""
    shape = {"qk": (Sq, Sk), "b11k": (B, 1, 1, Sk), "bhqk": (B, H, Sq, Sk), "1hqk": (1, H, Sq, Sk)}[layout]
    if kind == "bool":
        m = synth.uniform(shape, seed, 8) < 0.2
        m[..., 0] = True
    else:
        m = synth.to_bf16((synth.normal(shape, seed, 9) * 2.0).astype(np.float32))
    full = (1,) * (4 - len(shape)) + shape
    dense = [full[1] * full[2] * full[3], full[2] * full[3], full[3]]
    return m, [0 if full[i] == 1 else dense[i] for i in range(3)]


def _attn_ex(dev, q, k, v, scale, causal, mask, mstrides, cap, d, via_program=False):
    B, H, Sq, _ = q.shape
    Sk = k.shape[2]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    bo = dev.buffer(q.nbytes)
    kind = 0 if mask is None else 1 if mask.dtype == np.bool_ else 2
    bm = morok_amd.Buffer.from_numpy(mask.view(np.uint8) if kind == 1 else mask, dev.device_id) if kind else None
    if via_program:
        bits = lambda x: int(np.float32(x).view(np.uint32))
        dense = lambda rows: [H * rows * d, rows * d, d]
        params = [B, H, Sq, Sk, d, int(causal), bits(scale), bits(cap) if cap else 0, kind, 0, 0, 0, 0, 0,
                  *dense(Sq), *dense(Sk), *dense(Sk), *dense(Sq), *(mstrides if kind else [0, 0, 0])]
        prog = morok_amd.Program.builtin("flash_fwd_bf16_ext", params, dev.device_id)
        prog.execute([bo, bq, bk, bv, bm if kind else bq])
    else:
        ops.flash_attn_fwd_bf16_ex(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, causal, bm, kind, mstrides if kind else (0, 0, 0), cap,
                                   device_id=dev.device_id)
    return bo.copyout(np.uint16, q.shape)


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind,layout,cap", [(kind, layout, cap) for cap in (0.0, 1.5, 30.0)
                                             for kind, layout in (("none", None), ("bool", "qk"), ("bool", "b11k"), ("add", "bhqk"), ("add", "1hqk"))
                                             if kind != "none" or cap > 0.0])     # (no option at all is the plain kernel, covered above)
def test_flash_mask_and_softcap_vs_oracle(dev, oracle, d, causal, kind, layout, cap):
    """attn_mask (Bool / additive, several broadcast layouts) and softcap inside the fused kernel
    against the oracle's restatement of transformer.rs:96-132, ragged query and key counts, all
    three head dims; <= 2e-2 of the largest reference magnitude."""
    B, H, Sq, Sk = 2, 2, 200, 260
    q, k, v = (synth.normal_bf16((B, H, s, d), 41, i) for i, s in enumerate((Sq, Sk, Sk)))
    mask, mst = (None, None) if kind == "none" else _mask_for(kind, layout, B, H, Sq, Sk, 41)
    scale = 1.0 / np.sqrt(d)
    got = _attn_ex(dev, q, k, v, scale, causal, mask, mst, cap, d, via_program=(d == 128 and causal))
    ref = oracle.sdpa_bf16_ex(q, k, v, scale, causal=causal, mask=mask, softcap=cap)
    _check(got, ref)


def test_flash_mask_identities_and_empty_rows(dev, oracle):
    """A Bool tril mask, an additive mask that is -inf above the diagonal and is_causal agree with the
    plain causal kernel to the tolerance; an all-true mask is the plain kernel; a row with no key left
    is NaN and leaves the other rows alone; a key-padding mask equals attention over the kept keys."""
    B, H, S, d = 1, 2, 256, 128
    q, k, v = _inputs(B, H, S, S, seed=43)
    tril = np.tril(np.ones((S, S), bool))
    plain_causal = _attn(dev, q, k, v, SCALE, True)
    _check(_attn_ex(dev, q, k, v, SCALE, False, tril, [0, 0, S], 0.0, d), plain_causal)
    neg = synth.to_bf16(np.where(tril, 0.0, -np.inf).astype(np.float32))
    _check(_attn_ex(dev, q, k, v, SCALE, False, neg, [0, 0, S], 0.0, d), plain_causal)
    _check(_attn_ex(dev, q, k, v, SCALE, True, tril, [0, 0, S], 0.0, d), plain_causal)       # both at once
    _check(_attn_ex(dev, q, k, v, SCALE, False, np.ones((S, S), bool), [0, 0, S], 0.0, d), _attn(dev, q, k, v, SCALE, False))
    none = np.ones((S, S), bool)
    none[70] = False
    none[:, :64] |= False
    got = synth.from_bf16(_attn_ex(dev, q, k, v, SCALE, False, none, [0, 0, S], 0.0, d))
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, SCALE, mask=none))
    assert np.isnan(got[:, :, 70]).all() and np.isnan(ref[:, :, 70]).all()
    keep = np.delete(np.arange(S), 70)
    assert np.abs(got[:, :, keep] - ref[:, :, keep]).max() <= 2e-2 * np.abs(ref[:, :, keep]).max()
    # rows whose first key tiles are fully masked (a sliding window): the running maximum starts at -inf
    win = np.zeros((S, S), bool)
    for i in range(S):
        win[i, max(0, i - 20): i + 1] = True
    _check(_attn_ex(dev, q, k, v, SCALE, False, win, [0, 0, S], 0.0, d), oracle.sdpa_bf16_ex(q, k, v, SCALE, mask=win))
    pad = np.ones((B, 1, 1, S), bool)
    pad[..., 200:] = False
    _check(_attn_ex(dev, q, k, v, SCALE, False, pad, [S, 0, 0], 0.0, d),
           oracle.sdpa_bf16(q, k[:, :, :200], v[:, :, :200], SCALE, causal=False))


def test_flash_softcap_masked_scores_become_minus_cap(dev, oracle):
    """The reference caps after masking: with zero queries and keys every score is 0, a causally
    masked one -cap, so row i is the mean of v[0..i] and exp(-cap) times the rest."""
    S, d, cap = 128, 128, 0.75
    z = np.zeros((1, 1, S, d), np.uint16)
    v = synth.normal_bf16((1, 1, S, d), 44, 2)
    got = synth.from_bf16(_attn_ex(dev, z, z, v, 1.0, True, None, None, cap, d))
    vf = synth.from_bf16(v).astype(np.float64)[0, 0]
    w = np.where(np.tril(np.ones((S, S), bool)), 1.0, np.exp(-cap))
    ref = (w @ vf) / w.sum(1, keepdims=True)
    assert np.abs(got[0, 0] - ref).max() <= 2e-2 * np.abs(ref).max()
    _check(_attn_ex(dev, z, z, v, 1.0, True, None, None, cap, d), oracle.sdpa_bf16_ex(z, z, v, 1.0, causal=True, softcap=cap))


def test_flash_ex_argument_errors(dev):
    b = dev.buffer(4 * 128 * 2 * 8).ensure_allocated()
    with pytest.raises(MorokHipError):   # key count not a multiple of 4 with a mask
        ops.flash_attn_fwd_bf16_ex(b, b, b, b, 1, 1, 4, 6, 128, 1.0, False, b, 1, (0, 0, 8), 0.0)
    with pytest.raises(MorokHipError):   # mask stride not a multiple of 4
        ops.flash_attn_fwd_bf16_ex(b, b, b, b, 1, 1, 4, 8, 128, 1.0, False, b, 1, (0, 0, 6), 0.0)
    with pytest.raises(MorokHipError):   # negative softcap
        ops.flash_attn_fwd_bf16_ex(b, b, b, b, 1, 1, 4, 8, 128, 1.0, False, None, 0, (0, 0, 0), -1.0)
    with pytest.raises(MorokHipError):   # unknown mask kind
        ops.flash_attn_fwd_bf16_ex(b, b, b, b, 1, 1, 4, 8, 128, 1.0, False, b, 3, (0, 0, 8), 0.0)
