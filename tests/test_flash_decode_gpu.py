"""Attention for a handful of queries against a long key sequence (a decode step over a key/value
cache): Tensor::scaled_dot_product_attention (tensor/src/transformer.rs:78-137) called with a short q,
no causal rule.  Such shapes take the kernel that splits the key sequence over workgroups; parity
with the CPU oracle's SDPA on identical seeded inputs, tolerance as for the tiled kernel (<= 2e-2
max relative error for bf16 attention with f32 accumulation, max|gpu - ref| / max|ref|).  The
reference holds no value test at these shapes: pinned against the oracle, whose SDPA the reference's
own attention tests pin, and against the tiled kernel on the same keys."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, synth
from morok_amd._ffi import lib

pytestmark = pytest.mark.gpu


def _inputs(B, H, Sq, Sk, d, seed):
    return (synth.normal_bf16((B, H, Sq, d), seed, 0), synth.normal_bf16((B, H, Sk, d), seed, 1),
            synth.normal_bf16((B, H, Sk, d), seed, 2))


def _attn(dev, q, k, v, scale, causal=False, mode="abi"):
    """mode: "abi" (the C entry point, scratch from the allocator), "program" (builtin Program without
    scratch: one key range), "program_ws" (builtin Program with the scratch buffer the shape asks for)."""
    B, H, Sq, d = q.shape
    Sk = k.shape[2]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    guard = np.full((B * H * Sq + 3, d), 0x7FC0, np.uint16)  # rows behind the output must stay as they are
    bo = morok_amd.Buffer.from_numpy(guard, dev.device_id)
    if mode == "abi":
        ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, causal, dev.device_id)
    else:
        bits = int(np.float32(scale).view(np.uint32))
        ws = lib.mrk_hip_flash_attn_workspace_bytes(B, H, Sq, Sk, d, int(causal)) if mode == "program_ws" else 0
        if ws:
            prog = morok_amd.Program.builtin("flash_fwd_bf16", [B * H, Sq, Sk, d, int(causal), bits, ws], dev.device_id)
            assert prog.name.endswith("_splitkv")
            prog.execute([bo, bq, bk, bv, dev.buffer(ws)])
        else:
            prog = morok_amd.Program.builtin("flash_fwd_bf16", [B * H, Sq, Sk, d, int(causal), bits], dev.device_id)
            prog.execute([bo, bq, bk, bv])
    out = bo.copyout(np.uint16, guard.shape)
    assert np.all(out[B * H * Sq:] == 0x7FC0)
    return out[:B * H * Sq].reshape(q.shape)


def _check(o, ref, tight=8e-3):
    of, rf = synth.from_bf16(o), synth.from_bf16(ref)
    assert np.all(np.isfinite(of))
    err = np.abs(of - rf).max() / np.abs(rf).max()
    assert err <= 2e-2, err
    assert err <= tight, err  # in practice a few bf16 ulps of the row scale


SHAPES = [(1, 2, 1, 256), (2, 3, 1, 1000), (1, 4, 5, 777), (1, 1, 16, 4100), (1, 32, 1, 4096), (4, 8, 3, 2048), (3, 1, 16, 515),
          (2, 100, 1, 300), (1, 8, 2, 8192), (1, 4, 17, 777), (2, 2, 32, 1000), (1, 8, 24, 4096)]   # 17 and more: two query blocks


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("shape", SHAPES)
def test_decode_parity_shapes(dev, oracle, shape, d):
    B, H, Sq, Sk = shape
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=71)
    scale = float(d) ** -0.5
    ref = oracle.sdpa_bf16(q, k, v, scale, causal=False)
    o = _attn(dev, q, k, v, scale)
    _check(o, ref)
    # the same through a builtin Program, with the scratch buffer and without (one key range): the oracle's values
    # either way, and the same bits on every run
    o_ws = _attn(dev, q, k, v, scale, mode="program_ws")
    assert np.array_equal(o_ws, o)
    _check(_attn(dev, q, k, v, scale, mode="program"), ref)
    assert np.array_equal(_attn(dev, q, k, v, scale), o)


def test_decode_shapes_split_the_keys_where_pairs_are_few():
    ws = lib.mrk_hip_flash_attn_workspace_bytes
    assert ws(1, 32, 1, 4096, 128, 0) > 0 and ws(1, 8, 4, 8192, 64, 0) > 0 and ws(2, 16, 16, 2048, 256, 0) > 0
    assert ws(1, 32, 1, 4096, 128, 0) % (32 * 16 * 130 * 4) == 0  # whole slices of [pairs][16][D + 2] floats
    # the causal rule, many queries, few keys, no kernel for the head dim: no scratch
    for args in ((1, 32, 1, 4096, 128, 1), (1, 32, 33, 4096, 128, 0), (1, 32, 1, 255, 128, 0), (1, 32, 1, 4096, 96, 0), (0, 32, 1, 4096, 128, 0)):
        assert ws(*args) == 0, args
    # 512 pairs fill the chip by themselves, but should their heads share K and V (the launchers see the strides, this
    # query does not) they fold into as few as 32 pairs, which split their keys: a bounded reserve for that
    assert 0 < ws(16, 32, 1, 4096, 128, 0) <= 4 << 20
    assert ws(16, 32, 32, 4096, 128, 0) == 0   # 32 queries a head: nothing to fold
    assert ws(1, 32, 17, 4096, 128, 0) == 6 * 32 * 32 * 130 * 4   # 17 and more: 32 slots a pair (six key ranges, 32 pairs)


@pytest.mark.parametrize("d", [128, 64, 256])
def test_decode_special_cases(dev, d):
    B, H, Sk = 1, 3, 1234
    scale = float(d) ** -0.5
    q, k, v = _inputs(B, H, 2, Sk, d, seed=72)
    # uniform keys: every key scores the same -> the mean of V (to bf16 rounding of the weights)
    ku = np.ascontiguousarray(np.broadcast_to(k[:, :, :1], k.shape))
    o = synth.from_bf16(_attn(dev, q, ku, v, scale))
    mean = synth.from_bf16(v).astype(np.float64).mean(axis=2, keepdims=True)
    assert np.abs(o - mean).max() <= 1e-2
    # one key far above the rest: the output is that key's row of V, whichever range and chunk it sits in
    for hot in (0, 31, 32, 700, Sk - 1):
        kh = k.copy()
        kh[:, :, hot] = synth.to_bf16(synth.from_bf16(q[:, :, 0]) * 8.0)
        qq = q[:, :, :1]
        o = _attn(dev, qq, kh, v, 1.0)
        assert np.array_equal(o[:, :, 0], v[:, :, hot]), hot
    # identical V rows: softmax weights sum to one
    vu = np.ascontiguousarray(np.broadcast_to(v[:, :, :1], v.shape))
    o = synth.from_bf16(_attn(dev, q, k, vu, scale))
    assert np.abs(o - synth.from_bf16(vu[:, :, :2])).max() <= np.abs(synth.from_bf16(vu)).max() * 8e-3


def test_decode_rows_past_the_end_do_not_leak(dev, oracle):
    """A key count that is no multiple of the 32-key chunk: the chunk is filled up with copies of the last row,
    which must not count: with an infinity in that row of V the column is +inf (its weight times inf), not the
    NaN that a zero weight times a copy's infinity would add."""
    B, H, Sq, Sk, d = 1, 2, 1, 261, 128
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=73)
    v[:, :, Sk - 1, 5] = 0x7F80  # +inf
    scale = float(d) ** -0.5
    o = synth.from_bf16(_attn(dev, q, k, v, scale))
    ref = synth.from_bf16(oracle.sdpa_bf16(q, k, v, scale, causal=False))
    cols = np.arange(d) != 5
    assert np.all(np.isfinite(o[..., cols]))
    assert np.abs(o[..., cols] - ref[..., cols]).max() <= 2e-2 * np.abs(ref[..., cols]).max()
    assert np.all(np.isposinf(ref[..., 5])) and np.all(np.isposinf(o[..., 5]))


@pytest.mark.parametrize("d", [128, 64])
def test_decode_agrees_with_the_tiled_kernel(dev, d):
    """33 queries take the tiled kernel, their first 32 alone and their first 16 alone the split one (two query blocks,
    one): the same keys, the same values to the tolerance of either; a query's result does not depend on the block
    it sits in."""
    B, H, Sk = 2, 4, 3000
    scale = float(d) ** -0.5
    q, k, v = _inputs(B, H, 33, Sk, d, seed=74)
    tiled = _attn(dev, q, k, v, scale)
    split = _attn(dev, np.ascontiguousarray(q[:, :, :32]), k, v, scale)
    _check(split, tiled[:, :, :32], tight=1e-2)
    assert np.array_equal(_attn(dev, np.ascontiguousarray(q[:, :, :16]), k, v, scale), split[:, :, :16])
    assert np.array_equal(_attn(dev, np.ascontiguousarray(q[:, :, 16:32]), k, v, scale), split[:, :, 16:])
    # and the causal rule keeps the tiled kernel (a single query then sees key 0 only)
    o = _attn(dev, np.ascontiguousarray(q[:, :, :1]), k, v, scale, causal=True)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])


@pytest.mark.parametrize("via_program", [False, True])
def test_decode_over_a_cache_and_a_packed_projection(dev, oracle, via_program):
    """K and V as the first Sk rows of longer caches [B, H, Smax, D], q as a column slice of a packed [B, 1, 3 H D]
    projection, the output as a column slice of a wider matrix whose other columns must stay as they were."""
    B, H, Sq, Sk, Smax, d = 2, 4, 1, 1500, 2048, 128
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=75)
    hid = H * d
    packed = synth.normal_bf16((B, Sq, 3 * hid), 75, 5)
    packed[:, :, :hid] = q.transpose(0, 2, 1, 3).reshape(B, Sq, hid)
    ck, cv = synth.normal_bf16((B, H, Smax, d), 75, 6), synth.normal_bf16((B, H, Smax, d), 75, 7)
    ck[:, :, :Sk], cv[:, :, :Sk] = k, v
    wide = np.full((B, Sq, hid + 64), 0x7FC0, np.uint16)
    strides = [Sq * 3 * hid, d, 3 * hid, H * Smax * d, Smax * d, d, H * Smax * d, Smax * d, d, Sq * (hid + 64), d, hid + 64]
    offsets = [0, 0, 0, 32]
    bq, bk, bv, bo = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (packed, ck, cv, wide))
    scale = float(d) ** -0.5
    if via_program:
        bits = int(np.float32(scale).view(np.uint32))
        ws = lib.mrk_hip_flash_attn_workspace_bytes(B, H, Sq, Sk, d, 0)
        assert ws > 0
        prog = morok_amd.Program.builtin("flash_fwd_bf16_strided", [B, H, Sq, Sk, d, 0, bits, *offsets, *strides, ws], dev.device_id)
        assert prog.name.endswith("_splitkv")
        prog.execute([bo, bq, bk, bv, dev.buffer(ws)])
    else:
        ops.flash_attn_fwd_bf16_strided(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, strides, offsets, False, dev.device_id)
    o = bo.copyout(np.uint16, wide.shape)
    assert np.all(o[:, :, :32] == 0x7FC0) and np.all(o[:, :, 32 + hid:] == 0x7FC0)
    got = o[:, :, 32:32 + hid].reshape(B, Sq, H, d).transpose(0, 2, 1, 3)
    assert np.array_equal(got, _attn(dev, q, k, v, scale))
    _check(got, oracle.sdpa_bf16(q, k, v, scale, causal=False))


def test_decode_shared_keys_through_zero_strides(dev, oracle):
    B, H, Sq, Sk, d = 2, 3, 4, 900, 128
    q, _, _ = _inputs(B, H, Sq, Sk, d, seed=76)
    k1, v1 = synth.normal_bf16((1, 1, Sk, d), 76, 1), synth.normal_bf16((1, 1, Sk, d), 76, 2)
    strides = [H * Sq * d, Sq * d, d, 0, 0, d, 0, 0, d, H * Sq * d, Sq * d, d]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k1, v1))
    bo = morok_amd.Buffer.from_numpy(np.zeros_like(q), dev.device_id)
    scale = float(d) ** -0.5
    ops.flash_attn_fwd_bf16_strided(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, strides, [0, 0, 0, 0], False, dev.device_id)
    o = bo.copyout(np.uint16, q.shape)
    kb, vb = (np.ascontiguousarray(np.broadcast_to(t, (B, H, Sk, d))) for t in (k1, v1))
    assert np.array_equal(o, _attn(dev, q, kb, vb, scale))
    _check(o, oracle.sdpa_bf16(q, kb, vb, scale, causal=False))


@pytest.mark.parametrize("seed", range(12))
def test_decode_random_shapes(dev, oracle, seed):
    rng = np.random.default_rng(5000 + seed)
    d = int(rng.choice([64, 128, 256]))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 9))
    Sq, Sk = int(rng.integers(1, 33)), int(rng.integers(256, 3000))
    scale = float(rng.choice([float(d) ** -0.5, 0.05, 0.2]))
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=80 + seed)
    _check(_attn(dev, q, k, v, scale), oracle.sdpa_bf16(q, k, v, scale, causal=False))


def test_decode_through_the_tensor_api(dev, oracle):
    """One new token's attention over a cache, as a model's decode step writes it: q [B, H, 1, D] against the
    first Sk rows of the caches; one kernel launch entry, the scratch an intermediate of the plan."""
    from morok_amd import tensor as T, uop

    B, H, Sk, Smax, d = 1, 8, 2000, 2048, 128
    q, k, v = _inputs(B, H, 1, Sk, d, seed=77)
    ck, cv = synth.normal_bf16((B, H, Smax, d), 77, 6), synth.normal_bf16((B, H, Smax, d), 77, 7)
    ck[:, :, :Sk], cv[:, :, :Sk] = k, v
    tk = T.Tensor.from_numpy(ck, uop.BF16).try_shrink([(0, B), (0, H), (0, Sk), (0, d)])
    tv = T.Tensor.from_numpy(cv, uop.BF16).try_shrink([(0, B), (0, H), (0, Sk), (0, d)])
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(tk, tv)
    got = t.to_numpy()
    names = t.kernels()
    assert len(names) == 1 and names[0].startswith("flash_fwd_bf16_strided") and names[0].endswith("_splitkv"), names
    assert np.array_equal(got, _attn(dev, q, k, v, float(d) ** -0.5))
    _check(got, oracle.sdpa_bf16(q, k, v, float(d) ** -0.5, causal=False))


def test_decode_full_size_properties(dev):
    """A batch of 16 sequences of 2048 cached keys, 32 heads: the oracle would take minutes, so size-independent
    properties: uniform keys give the mean of V, and the result does not depend on the batch a sequence sits in."""
    B, H, Sk, d = 16, 32, 2048, 128
    scale = float(d) ** -0.5
    q, k, v = _inputs(B, H, 1, Sk, d, seed=78)
    o = _attn(dev, q, k, v, scale)
    one = _attn(dev, q[5:6], k[5:6], v[5:6], scale)  # 32 pairs: split keys; 512 pairs: one range each
    _check(one, o[5:6])
    ku = np.ascontiguousarray(np.broadcast_to(k[:, :, :1], k.shape))
    ou = synth.from_bf16(_attn(dev, q, ku, v, scale))
    mean = synth.from_bf16(v).astype(np.float64).mean(axis=2, keepdims=True)
    assert np.abs(ou - mean).max() <= 1e-2


# ---------------------------------------------------------------- attn_mask over a decode shape
def _mask_for(kind, layout, B, H, Sq, Sk, seed, keep=0.6):
    """(host array for the oracle, element strides per batch / head / row) of a mask broadcastable to [B, H, Sq, Sk]."""
    shape = {"b11k": (B, 1, 1, Sk), "bhqk": (B, H, Sq, Sk), "1hqk": (1, H, Sq, Sk), "qk": (Sq, Sk)}[layout]
    if kind == "bool":
        m = synth.uniform(shape, seed, 8) < keep
        m[..., 0] = True  # no empty row
    else:
        m = synth.to_bf16((synth.normal(shape, seed, 9) * 2.0).astype(np.float32))
    full = (1,) * (4 - len(shape)) + shape
    dense = [full[1] * full[2] * full[3], full[2] * full[3], full[3]]
    return m, [0 if full[i] == 1 else dense[i] for i in range(3)]


def _attn_masked(dev, q, k, v, scale, mask, mstrides, mode="abi", cap=0.0):
    B, H, Sq, d = q.shape
    Sk = k.shape[2]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    bo = dev.buffer(q.nbytes)
    kind = 0 if mask is None else 1 if mask.dtype == np.bool_ else 2
    bm = morok_amd.Buffer.from_numpy(mask.view(np.uint8) if kind == 1 else mask, dev.device_id) if kind else bq
    mstrides = mstrides if kind else [0, 0, 0]
    if mode == "abi":
        ops.flash_attn_fwd_bf16_ex(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, False, bm if kind else None, kind, mstrides, cap,
                                   device_id=dev.device_id)
    else:
        bits = int(np.float32(scale).view(np.uint32))
        cbits = int(np.float32(cap).view(np.uint32)) if cap else 0
        dense = lambda rows: [H * rows * d, rows * d, d]
        params = [B, H, Sq, Sk, d, 0, bits, cbits, kind, 0, 0, 0, 0, 0, *dense(Sq), *dense(Sk), *dense(Sk), *dense(Sq), *mstrides]
        ws = lib.mrk_hip_flash_attn_workspace_bytes(B, H, Sq, Sk, d, 0) if mode == "program_ws" else 0
        if ws:
            prog = morok_amd.Program.builtin("flash_fwd_bf16_ext", params + [ws], dev.device_id)
            assert prog.name.endswith("_splitkv")
            prog.execute([bo, bq, bk, bv, bm, dev.buffer(ws)])
        else:
            morok_amd.Program.builtin("flash_fwd_bf16_ext", params, dev.device_id).execute([bo, bq, bk, bv, bm])
    return bo.copyout(np.uint16, q.shape)


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("kind,layout", [("bool", "b11k"), ("bool", "bhqk"), ("add", "1hqk"), ("add", "bhqk"), ("bool", "qk")])
@pytest.mark.parametrize("shape", [(2, 4, 1, 1000), (1, 32, 1, 4096), (3, 2, 5, 516), (1, 2, 16, 2052), (1, 2, 20, 516)])
def test_decode_mask_vs_oracle(dev, oracle, shape, kind, layout, d):
    """attn_mask (transformer.rs:112-125) over decode shapes: a key-padding mask [B, 1, 1, Sk] is what a batch of
    sequences of different lengths decodes with.  The oracle's restatement, through the C entry point and through a
    Program with and without the scratch buffer."""
    B, H, Sq, Sk = shape
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=91)
    mask, mst = _mask_for(kind, layout, B, H, Sq, Sk, 91)
    scale = float(d) ** -0.5
    ref = oracle.sdpa_bf16_ex(q, k, v, scale, causal=False, mask=mask, softcap=0.0)
    got = _attn_masked(dev, q, k, v, scale, mask, mst)
    _check(got, ref)
    assert np.array_equal(_attn_masked(dev, q, k, v, scale, mask, mst, mode="program_ws"), got)
    _check(_attn_masked(dev, q, k, v, scale, mask, mst, mode="program"), ref)


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("cap", [1.5, 30.0])
@pytest.mark.parametrize("kind,layout", [("none", None), ("bool", "b11k"), ("add", "bhqk")])
def test_decode_softcap_vs_oracle(dev, oracle, kind, layout, cap, d):
    """softcap (transformer.rs:128-132) inside the split kernel, alone and after a mask: a masked score becomes -cap and
    still takes part, as in the reference's graph."""
    B, H, Sq, Sk = 2, 4, 3, 1540
    q, k, v = _inputs(B, H, Sq, Sk, d, seed=94)
    mask, mst = (None, None) if kind == "none" else _mask_for(kind, layout, B, H, Sq, Sk, 94)
    scale = float(d) ** -0.5
    ref = oracle.sdpa_bf16_ex(q, k, v, scale, causal=False, mask=mask, softcap=cap)
    got = _attn_masked(dev, q, k, v, scale, mask, mst, cap=cap)
    _check(got, ref)
    assert np.array_equal(_attn_masked(dev, q, k, v, scale, mask, mst, mode="program_ws", cap=cap), got)
    _check(_attn_masked(dev, q, k, v, scale, mask, mst, mode="program", cap=cap), ref)
    if kind == "bool":
        # every key masked out under a cap: all scores -cap, the mean of V (not NaN)
        none = np.zeros_like(mask)
        o = synth.from_bf16(_attn_masked(dev, q, k, v, scale, none, mst, cap=cap))
        mean = synth.from_bf16(v).astype(np.float64).mean(axis=2, keepdims=True)
        assert np.abs(o - mean).max() <= 1e-2


def test_decode_mask_ragged_lengths_and_empty_ranges(dev, oracle):
    """Sequences of different lengths in one batch (keys past a sequence's length masked out): whole chunks, whole
    waves' shares and whole key ranges without a visible key must weigh nothing; the result is the unmasked attention
    over each sequence's own keys.  A sequence with no visible key at all is NaN, as the reference's softmax over
    -inf only is."""
    B, H, Sq, Smax, d = 4, 8, 1, 4096, 128
    lengths = [4096, 1, 700, 33]
    q, k, v = _inputs(B, H, Sq, Smax, d, seed=92)
    mask = np.zeros((B, 1, 1, Smax), np.bool_)
    for b, n in enumerate(lengths):
        mask[b, ..., :n] = True
    scale = float(d) ** -0.5
    assert lib.mrk_hip_flash_attn_workspace_bytes(B, H, Sq, Smax, d, 0) > 0   # 32 pairs: several key ranges
    got = _attn_masked(dev, q, k, v, scale, mask, [Smax, 0, 0])
    _check(got, oracle.sdpa_bf16_ex(q, k, v, scale, causal=False, mask=mask, softcap=0.0))
    for b, n in enumerate(lengths):
        if n >= 256:  # the same keys without a mask, through the same kernel family
            alone = _attn(dev, q[b:b + 1], np.ascontiguousarray(k[b:b + 1, :, :n]), np.ascontiguousarray(v[b:b + 1, :, :n]), scale)
            _check(got[b:b + 1], alone)
    assert np.array_equal(got[1, :, 0], v[1, :, 0])  # one visible key: its row of V
    # additive -inf does the same as Bool false
    add = np.where(mask, np.float32(0), np.float32(-np.inf)).astype(np.float32)
    got_add = _attn_masked(dev, q, k, v, scale, synth.to_bf16(add), [Smax, 0, 0])
    _check(got_add, got)
    # a sequence without any visible key
    mask[2] = False
    got = synth.from_bf16(_attn_masked(dev, q, k, v, scale, mask, [Smax, 0, 0]))
    assert np.all(np.isnan(got[2])) and np.all(np.isfinite(got[[0, 1, 3]]))


def test_decode_mask_through_the_tensor_api(dev, oracle):
    from morok_amd import tensor as T, uop

    B, H, Sk, d = 2, 8, 2048, 128
    q, k, v = _inputs(B, H, 1, Sk, d, seed=93)
    mask, _ = _mask_for("bool", "b11k", B, H, 1, Sk, 93)
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16), T.Tensor.from_numpy(v, uop.BF16),
                                                                      attn_mask=T.Tensor.from_numpy(mask))
    got = t.to_numpy()
    names = [n for n in t.kernels() if n.startswith("flash_fwd")]
    assert len(names) == 1 and names[0].startswith("flash_fwd_bf16_ext_bool") and names[0].endswith("_splitkv"), t.kernels()
    _check(got, oracle.sdpa_bf16_ex(q, k, v, float(d) ** -0.5, causal=False, mask=mask, softcap=0.0))


# ---------------------------------------------------------------- heads that share their keys and values
def _attn_shared(dev, q, k1, v1, scale, mask=None, mstrides=None):
    """q [B, H, Sq, d] against k1 / v1 [B, 1, Sk, d] shared by the H heads of a batch (head stride 0: what `expand` over
    the head axis hands over), through the strided entry point, or the extended one with a mask."""
    B, H, Sq, d = q.shape
    Sk = k1.shape[2]
    strides = [H * Sq * d, Sq * d, d, Sk * d, 0, d, Sk * d, 0, d, H * Sq * d, Sq * d, d]
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k1, v1))
    guard = np.full((B * H * Sq + 2, d), 0x7FC0, np.uint16)
    bo = morok_amd.Buffer.from_numpy(guard, dev.device_id)
    if mask is None:
        ops.flash_attn_fwd_bf16_strided(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, strides, [0, 0, 0, 0], False, dev.device_id)
    else:
        kind = 1 if mask.dtype == np.bool_ else 2
        bm = morok_amd.Buffer.from_numpy(mask.view(np.uint8) if kind == 1 else mask, dev.device_id)
        ops.flash_attn_fwd_bf16_ex(bq, bk, bv, bo, B, H, Sq, Sk, d, scale, False, bm, kind, mstrides, 0.0, strides=strides,
                                   device_id=dev.device_id)
    out = bo.copyout(np.uint16, guard.shape)
    assert np.all(out[B * H * Sq:] == 0x7FC0)
    return out[:B * H * Sq].reshape(q.shape)


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("shape", [(2, 8, 1, 3000), (1, 16, 1, 4096), (3, 4, 4, 777), (8, 4, 1, 1024), (2, 5, 3, 515), (1, 9, 2, 600),
                                   (2, 32, 1, 2048), (1, 12, 2, 1000), (1, 7, 3, 300), (1, 64, 1, 1000), (1, 11, 3, 300)])
def test_decode_heads_sharing_keys_are_folded(dev, oracle, shape, d):
    """Multi-query attention (and grouped-query attention with the groups as batches): the heads of a batch read the
    same K and V; runs of consecutive heads become query slots of one pass over the keys, as many as give at most 32
    slots (64 heads: two runs of 32; 12 heads of two rows: one run of 24 slots; 7 heads of three rows: one run of 21;
    11 of three: head by head, 33 slots being too many and 11 having no smaller divisor but 1).
    The oracle's values over broadcast copies."""
    B, H, Sq, Sk = shape
    q = synth.normal_bf16((B, H, Sq, d), 95, 0)
    k1, v1 = synth.normal_bf16((B, 1, Sk, d), 95, 1), synth.normal_bf16((B, 1, Sk, d), 95, 2)
    kb, vb = (np.ascontiguousarray(np.broadcast_to(t, (B, H, Sk, d))) for t in (k1, v1))
    scale = float(d) ** -0.5
    got = _attn_shared(dev, q, k1, v1, scale)
    ref = oracle.sdpa_bf16(q, kb, vb, scale, causal=False)
    _check(got, ref)
    _check(got, _attn(dev, q, kb, vb, scale), tight=1e-2)   # the unfolded kernel over copies
    assert np.array_equal(_attn_shared(dev, q, k1, v1, scale), got)


@pytest.mark.parametrize("H", [8, 12, 32])
def test_decode_folded_heads_under_masks(dev, oracle, H):
    B, Sq, Sk, d = 2, (1 if H == 32 else 2), 2052, 128
    q = synth.normal_bf16((B, H, Sq, d), 96, 0)
    k1, v1 = synth.normal_bf16((B, 1, Sk, d), 96, 1), synth.normal_bf16((B, 1, Sk, d), 96, 2)
    kb, vb = (np.ascontiguousarray(np.broadcast_to(t, (B, H, Sk, d))) for t in (k1, v1))
    scale = float(d) ** -0.5
    for kind, layout in (("bool", "b11k"), ("bool", "bhqk"), ("add", "1hqk")):
        mask, mst = _mask_for(kind, layout, B, H, Sq, Sk, 96)
        got = _attn_shared(dev, q, k1, v1, scale, mask, mst)
        _check(got, oracle.sdpa_bf16_ex(q, kb, vb, scale, causal=False, mask=mask, softcap=0.0))


def test_decode_folded_heads_through_the_tensor_api(dev, oracle):
    """K and V of one head expanded over the query heads: read in place with a zero head stride, the heads folded."""
    from morok_amd import tensor as T, uop

    B, H, Sk, d = 2, 8, 2048, 128
    q = synth.normal_bf16((B, H, 1, d), 97, 0)
    k1, v1 = synth.normal_bf16((B, 1, Sk, d), 97, 1), synth.normal_bf16((B, 1, Sk, d), 97, 2)
    tk = T.Tensor.from_numpy(k1, uop.BF16).try_expand([B, H, Sk, d])
    tv = T.Tensor.from_numpy(v1, uop.BF16).try_expand([B, H, Sk, d])
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(tk, tv)
    got = t.to_numpy()
    names = t.kernels()
    assert len(names) == 1 and names[0].startswith("flash_fwd_bf16_strided"), names
    kb, vb = (np.ascontiguousarray(np.broadcast_to(x, (B, H, Sk, d))) for x in (k1, v1))
    _check(got, oracle.sdpa_bf16(q, kb, vb, float(d) ** -0.5, causal=False))
    assert np.array_equal(got, _attn_shared(dev, q, k1, v1, float(d) ** -0.5))


def test_decode_attention_in_a_replayed_graph(dev, oracle):
    """The split kernel and its merge as two kernel nodes of a plan recorded into a HIP graph, the scratch an
    intermediate of the plan: every replay, with eager work and synchronisations in between and new queries each
    time, gives what the eager launches give."""
    from morok_amd import tensor as T, uop

    B, H, Sk, d = 1, 8, 2048, 128
    q, k, v = _inputs(B, H, 2, Sk, d, seed=98)
    tq = T.Tensor.from_numpy(q, uop.BF16)
    out = tq.scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16), T.Tensor.from_numpy(v, uop.BF16))
    plan = out.prepare()
    assert out.kernels()[0].endswith("_splitkv")
    qbuf = tq.buffer()

    def result():
        dev.synchronize()
        return out.buffer().copyout(np.uint16, q.shape).copy()

    plan.execute()
    _check(result(), oracle.sdpa_bf16(q, k, v, float(d) ** -0.5, causal=False))
    for i in range(4):
        qi = synth.normal_bf16(q.shape, 99, i)
        qbuf.copyin(qi)
        plan.execute()
        want = result()
        out.buffer().copyin(np.zeros(q.size, np.uint16))   # the replay must rewrite it
        plan.execute_graph()
        got = result()
        assert np.array_equal(got, want), i
        _check(got, oracle.sdpa_bf16(qi, k, v, float(d) ** -0.5, causal=False))
        x = synth.normal((64, 512), 5, i, sigma=1.0)       # unrelated eager work between the replays
        bx = morok_amd.Buffer.from_numpy(x, dev.device_id)
        ops.softmax_f32(bx, dev.buffer(x.nbytes), 64, 512, dev.device_id)
        dev.synchronize()
