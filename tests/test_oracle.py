"""Pins the CPU oracle (oracle/morok_cpu_oracle.c) before anything is compared with it:
against the known answers held by the reference's own tests (tests/golden/
reference_known_answers.json) and against what the mathematics fixes (float64 closed forms,
invariants, special cases).  Runs without a GPU."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from morok_amd import synth

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


# ------------------------------------------------------------------ matmul (C1)
def test_matmul_reference_small_cases(oracle):
    for key in ("matmul_2x2", "matmul_3x3"):
        g = GOLD[key]
        c = oracle.matmul_f32(np.array(g["a"], np.float32), np.array(g["b"], np.float32))
        assert np.abs(c - np.array(g["expected"], np.float32)).max() < g["tol"]


def test_matmul_reference_vector_cases(oracle):
    """Dot product, vector x matrix and matrix x vector of the reference's tests, through the
    oracle's matmul with the vector as a one-row / one-column matrix."""
    g = GOLD["matmul_dot_1d"]
    c = oracle.matmul_f32(np.array([g["a"]], np.float32), np.array(g["b"], np.float32).reshape(-1, 1))
    assert abs(float(c[0, 0]) - g["expected"]) < g["tol"]
    g = GOLD["matmul_vector_matrix"]
    c = oracle.matmul_f32(np.array([g["v"]], np.float32), np.array(g["m"], np.float32))
    assert np.abs(c[0] - np.array(g["expected"], np.float32)).max() < g["tol"]
    g = GOLD["matmul_matrix_vector"]
    c = oracle.matmul_f32(np.array(g["m"], np.float32), np.array(g["v"], np.float32).reshape(-1, 1))
    assert np.abs(c[:, 0] - np.array(g["expected"], np.float32)).max() < g["tol"]


@pytest.mark.parametrize("size,tol", [tuple(x) for x in GOLD["matmul_square_closed_form"]["sizes_tol"]])
def test_matmul_reference_square_generators(oracle, size, tol):
    x = np.arange(size * size)
    a = ((x % 31).astype(np.float32) * np.float32(0.05) - np.float32(0.8)).reshape(size, size)
    b = ((x % 37).astype(np.float32) * np.float32(0.04) - np.float32(0.7)).reshape(size, size)
    c = oracle.matmul_f32(a, b)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    err = np.abs(c - ref).max()
    assert err < tol  # the reference's tolerance against ndarray dot
    assert err < 1e-4 * np.abs(ref).max() + 1e-3  # and the much tighter bound the math supports


@pytest.mark.parametrize("m,k,n,tol", [tuple(x) for x in GOLD["matmul_nonsquare_closed_form"]["mkn_tol"]])
def test_matmul_reference_nonsquare_generators(oracle, m, k, n, tol):
    a = ((np.arange(m * k) % 41).astype(np.float32) * np.float32(0.04) - np.float32(0.8)).reshape(m, k)
    b = ((np.arange(k * n) % 43).astype(np.float32) * np.float32(0.035) - np.float32(0.7)).reshape(k, n)
    c = oracle.matmul_f32(a, b)
    assert c.shape == (m, n)
    assert np.abs(c - a.astype(np.float64) @ b.astype(np.float64)).max() < min(tol, 1e-3)


def test_matmul_ones_and_sincos(oracle):
    for size in GOLD["matmul_ones"]["sizes"]:
        c = oracle.matmul_f32(np.ones((size, size), np.float32), np.ones((size, size), np.float32))
        assert np.all(c == size)
    x = np.arange(64 * 64, dtype=np.float32)
    a = np.sin(x * np.float32(0.01)).reshape(64, 64)
    b = np.cos(x * np.float32(0.02)).reshape(64, 64)
    assert np.abs(oracle.matmul_f32(a, b) - a.astype(np.float64) @ b.astype(np.float64)).max() < 1e-4


def test_matmul_operand_order_and_threads(oracle):
    # a transposed operand or swapped index would fail this: A is not square, B is not symmetric
    a = synth.uniform((37, 53), 11, 0)
    b = synth.uniform((53, 29), 11, 1)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    for t in (1, 2, 5):
        assert np.abs(oracle.matmul_f32(a, b, threads=t) - ref).max() < 2e-5


# ------------------------------------------------------------------ thread rule
def test_thread_rule(oracle):
    # schedule/src/optimizer/heuristics.rs:485-535
    assert oracle.thread_count(1024 * 1024 * 1024, 1024, 8) == 8
    assert oracle.thread_count(1024 * 1024 * 1024, 1024, 64) == 32
    assert oracle.thread_count(1024 * 1024 * 1024, 1000, 16) == 8  # 16 and 12 do not divide 1000
    assert oracle.thread_count(131072 * 2 - 1, 1024, 16) == 1  # not enough work for 2 threads
    assert oracle.thread_count(131072 * 3, 9, 16) == 3
    assert oracle.thread_count(10**9, 7, 16) == 1
    assert oracle.thread_count(10**9, 1024, 1) == 1


# ------------------------------------------------------------------ softmax (C2)
def _softmax64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def test_softmax_vs_float64_and_invariants(oracle):
    x = synth.normal((64, 1000), 2, 0, sigma=2.0)
    y = oracle.softmax_f32(x)
    ref = _softmax64(x)
    assert np.abs(y - ref).max() / ref.max() < 1e-6
    assert np.all(np.abs(y / ref - 1.0) < 1e-5)
    # reference-held invariants: sums to one within 1e-4, 0 < p <= 1
    assert np.abs(y.sum(-1, dtype=np.float64) - 1.0).max() < GOLD["softmax_invariants"]["row_sum_tol"]
    assert np.all(y > 0) and np.all(y <= 1)
    # shift invariance and argmax preservation
    y2 = oracle.softmax_f32(x + np.float32(3.0))
    assert np.abs(y2 - y).max() < 1e-6
    assert np.all(y.argmax(-1) == x.argmax(-1))


def test_softmax_tiny_bruteforce_and_edges(oracle):
    y = oracle.softmax_f32(np.array([[0.0, np.log(3.0)]], np.float32))
    assert np.allclose(y, [[0.25, 0.75]], atol=1e-6)
    y = oracle.softmax_f32(np.array([[5.0]], np.float32))
    assert y[0, 0] == 1.0
    y = oracle.softmax_f32(np.array([[1e4, -1e4, 1e4]], np.float32))  # no overflow with max-subtraction
    assert np.allclose(y, [[0.5, 0.0, 0.5]])
    y = oracle.softmax_f32(np.array([[-np.inf, 0.0, 0.0]], np.float32))
    assert np.allclose(y, [[0.0, 0.5, 0.5]])


# ------------------------------------------------------------------ bf16 helpers
def test_bf16_rounding_matches_definition():
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.1415927, 65504.0, 1e-40, np.inf], np.float32)
    b = synth.to_bf16(x)
    back = synth.from_bf16(b)
    # 1 + 2^-8 is a tie between 1.0 and 1 + 2^-7 -> even mantissa (1.0); 1 + 3*2^-8 ties up
    assert back[0] == 1.0 and back[1] == 1.0 and back[2] == np.float32(1.015625)
    assert back[3] == -2.5
    assert abs(back[4] - 3.1415927) <= 2**-7
    assert np.isinf(back[7])
    assert np.isnan(synth.from_bf16(synth.to_bf16(np.array([np.nan], np.float32)))[0])


# ------------------------------------------------------------------ bf16 GEMM (C3)
def test_gemm_bf16_vs_float64(oracle):
    a = synth.normal_bf16((96, 160), 3, 0)
    b = synth.normal_bf16((160, 72), 3, 1)
    c = synth.from_bf16(oracle.gemm_bf16(a, b))
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    # f32 accumulation of exact products, one rounding to bf16 (2^-9 relative)
    assert np.all(np.abs(c - ref) <= np.abs(ref) * 2**-8 + 1e-4)
    lit = synth.from_bf16(oracle.gemm_bf16(a, b, literal=True))
    assert np.abs(lit - ref).max() / np.abs(ref).max() < 2e-2  # the literal graph stays inside the tolerance


def test_gemm_bf16_special_cases(oracle):
    n = 64
    eye = synth.to_bf16(np.eye(n, dtype=np.float32))
    a = synth.normal_bf16((n, n), 3, 2)
    assert np.array_equal(oracle.gemm_bf16(a, eye), a)
    assert np.array_equal(oracle.gemm_bf16(eye, a), a)
    perm = np.eye(n, dtype=np.float32)[:, ::-1].copy()
    assert np.array_equal(oracle.gemm_bf16(a, synth.to_bf16(perm)), a[:, ::-1])
    ones = synth.to_bf16(np.ones((n, 2 * n), np.float32))
    c = synth.from_bf16(oracle.gemm_bf16(ones, synth.to_bf16(np.ones((2 * n, n), np.float32))))
    assert np.all(c == 2 * n)


# ------------------------------------------------------------------ SDPA (C4)
def _sdpa64(q, k, v, scale, causal):
    q, k, v = (t.astype(np.float64) for t in (q, k, v))
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    if causal:
        sq, sk = s.shape[-2:]
        s = np.where(np.tril(np.ones((sq, sk), bool)), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", p, v)


def test_sdpa_reference_causal_row0(oracle):
    g = GOLD["sdpa_causal_row0"]
    q = np.array(g["q"], np.float32).reshape(1, 1, 3, 2)
    v = np.array(g["v"], np.float32).reshape(1, 1, 3, 2)
    o = oracle.sdpa_f32(q, q, v, 1.0 / np.sqrt(2.0), causal=True)
    assert np.abs(o[0, 0, 0] - np.array(g["expected_row0"])).max() < g["tol"]
    ref = _sdpa64(q, q, v, 1.0 / np.sqrt(2.0), True)
    assert np.abs(o - ref).max() < 1e-6


def test_sdpa_bf16_vs_float64_and_special_cases(oracle):
    B, H, S, D = 2, 3, 80, 32
    q = synth.normal_bf16((B, H, S, D), 4, 0)
    k = synth.normal_bf16((B, H, S, D), 4, 1)
    v = synth.normal_bf16((B, H, S, D), 4, 2)
    scale = 1.0 / np.sqrt(D)
    for causal in (True, False):
        o = synth.from_bf16(oracle.sdpa_bf16(q, k, v, scale, causal=causal))
        ref = _sdpa64(synth.from_bf16(q), synth.from_bf16(k), synth.from_bf16(v), scale, causal)
        assert np.abs(o - ref).max() < 2e-2 * np.abs(ref).max()
    o = oracle.sdpa_bf16(q, k, v, scale, causal=True)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])  # first causal row attends to key 0 only
    # uniform K: every visible key has the same score -> causal running mean of V
    k1 = np.broadcast_to(k[:, :, :1], k.shape).copy()
    o = synth.from_bf16(oracle.sdpa_bf16(q, k1, v, scale, causal=True))
    run = np.cumsum(synth.from_bf16(v).astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert np.abs(o - run).max() < 2e-2
    # S = 1
    o = oracle.sdpa_bf16(q[:, :, :1], k[:, :, :1], v[:, :, :1], scale, causal=True)
    assert np.array_equal(o, v[:, :, :1])
    # the row-parallel timing variant computes the same thing
    o_rows = oracle.sdpa_bf16_rows(q[0, 0], k[0, 0], v[0, 0], scale, causal=True)
    assert np.array_equal(o_rows, oracle.sdpa_bf16(q[:1, :1], k[:1, :1], v[:1, :1], scale, causal=True)[0, 0])
    # literal reference dtype flow (bf16 softmax) stays within the stated tolerance of the policy
    lit = synth.from_bf16(oracle.sdpa_bf16(q, k, v, scale, causal=True, policy=1))
    pol = synth.from_bf16(oracle.sdpa_bf16(q, k, v, scale, causal=True, policy=0))
    assert np.abs(lit - pol).max() < 6e-2 * np.abs(pol).max()


def _sdpa64_ex(q, k, v, scale, causal, mask_add=None, cap=0.0):
    """float64 restatement of transformer.rs:96-132: scale, causal where(-inf), additive mask, softcap
    AFTER the masks, softmax over every key."""
    q, k, v = (t.astype(np.float64) for t in (q, k, v))
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    if causal:
        sq, sk = s.shape[-2:]
        s = np.where(np.tril(np.ones((sq, sk), bool)), s, -np.inf)
    if mask_add is not None:
        s = s + mask_add
    if cap > 0:
        s = np.tanh(s / cap) * cap
    with np.errstate(invalid="ignore"):
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", p, v)


def test_sdpa_mask_and_softcap_closed_forms_identities_and_float64(oracle):
    """orc_sdpa_bf16_ex has no values to match in the reference's tests (its softcap test only asks
    for finite outputs), so it is pinned here: the reference's softcap case in closed form, masks
    that must reproduce the causal path bit for bit, the -cap (not -inf) a masked score turns into
    under a softcap, a fully masked row, and float64 on random inputs for every combination."""
    g = GOLD["sdpa_softcap_finite"]
    q = synth.to_bf16(np.array(g["q"], np.float32))
    v = synth.to_bf16(np.array(g["v"], np.float32))
    o = synth.from_bf16(oracle.sdpa_bf16_ex(q, q, v, 1.0 / np.sqrt(2.0), softcap=g["softcap"]))
    assert np.isfinite(o).all()
    # scores 70.7 / 0 -> tanh(70.7) = 1, tanh(0) = 0 -> softmax([1, 0]) = [e, 1] / (e + 1)
    w = np.e / (np.e + 1.0)
    assert np.abs(o - np.array([[[[w, 1 - w], [1 - w, w]]]])).max() < 4e-3          # bf16 output rounding
    B, H, Sq, Sk, D = 2, 3, 40, 56, 32
    qb, kb, vb = (synth.normal_bf16((B, H, s_, D), 31, i) for i, s_ in enumerate((Sq, Sk, Sk)))
    qf, kf, vf = (synth.from_bf16(t) for t in (qb, kb, vb))
    scale = 1.0 / np.sqrt(D)
    plain = oracle.sdpa_bf16_ex(qb, kb, vb, scale)
    sq_k = oracle.sdpa_bf16(qb[:, :, :, :], kb[:, :, :Sq], vb[:, :, :Sq], scale, causal=True)
    tril = np.tril(np.ones((Sq, Sq), bool))
    # identities, bit for bit: no options = the plain function; a True mask and a zero mask change nothing;
    # a Bool tril mask and an additive -inf-above-the-diagonal mask are the causal path
    assert np.array_equal(plain, oracle.sdpa_bf16(qb, kb, vb, scale, causal=False))
    assert np.array_equal(plain, oracle.sdpa_bf16_ex(qb, kb, vb, scale, mask=np.ones((Sq, Sk), bool)))
    assert np.array_equal(plain, oracle.sdpa_bf16_ex(qb, kb, vb, scale, mask=np.zeros((B, 1, Sq, Sk), np.uint16)))
    assert np.array_equal(sq_k, oracle.sdpa_bf16_ex(qb, kb[:, :, :Sq], vb[:, :, :Sq], scale, causal=True))
    assert np.array_equal(sq_k, oracle.sdpa_bf16_ex(qb, kb[:, :, :Sq], vb[:, :, :Sq], scale, mask=tril))
    neg = synth.to_bf16(np.where(tril, 0.0, -np.inf).astype(np.float32))
    assert np.array_equal(sq_k, oracle.sdpa_bf16_ex(qb, kb[:, :, :Sq], vb[:, :, :Sq], scale, mask=neg))
    # per-batch key padding mask [B, 1, 1, Sk] = attention over the kept keys only
    keep = np.ones((B, 1, 1, Sk), bool)
    keep[0, :, :, 40:] = False
    keep[1, :, :, :7] = False
    got = oracle.sdpa_bf16_ex(qb, kb, vb, scale, mask=keep)
    assert np.array_equal(got[0], oracle.sdpa_bf16(qb[:1], kb[:1, :, :40], vb[:1, :, :40], scale, causal=False)[0])
    assert np.array_equal(got[1], oracle.sdpa_bf16(qb[1:], kb[1:, :, 7:], vb[1:, :, 7:], scale, causal=False)[0])
    # a row with no key left is NaN (softmax over -inf only); the other rows are untouched
    none = np.ones((Sq, Sk), bool)
    none[5] = False
    got = synth.from_bf16(oracle.sdpa_bf16_ex(qb, kb, vb, scale, mask=none))
    assert np.isnan(got[:, :, 5]).all() and np.array_equal(np.delete(got, 5, 2), np.delete(synth.from_bf16(plain), 5, 2))
    # softcap after the masks: with two keys, zero queries and key 1 masked, the scores are [0, -cap],
    # so row 0 is (v0 + exp(-cap) v1) / (1 + exp(-cap)), not v0
    z = np.zeros((1, 1, 2, 8), np.uint16)
    v2 = synth.to_bf16(np.array([[1.0] * 8, [3.0] * 8], np.float32).reshape(1, 1, 2, 8))
    for cap in (0.5, 2.0):
        got = synth.from_bf16(oracle.sdpa_bf16_ex(z, z, v2, 1.0, causal=True, softcap=cap))
        e = np.exp(-cap)
        assert abs(got[0, 0, 0, 0] - (1.0 + 3.0 * e) / (1.0 + e)) < 1e-2 and abs(got[0, 0, 1, 0] - 2.0) < 1e-2
    # float64 on random inputs, every combination
    add = synth.from_bf16(synth.normal_bf16((B, H, Sq, Sk), 31, 7)).astype(np.float64) * 2.0
    addb = synth.to_bf16(add.astype(np.float32))
    add = synth.from_bf16(addb).astype(np.float64)
    boolm = synth.uniform((H, Sq, Sk), 31, 8) < 0.6
    boolm[..., 0] = True                                                           # no empty rows
    for causal in (False, True):
        for cap in (0.0, 1.5, 30.0):
            for kind in ("none", "bool", "add"):
                m = None if kind == "none" else boolm if kind == "bool" else addb
                m64 = None if kind == "none" else np.where(boolm, 0.0, -np.inf)[None] if kind == "bool" else add
                got = synth.from_bf16(oracle.sdpa_bf16_ex(qb, kb, vb, scale, causal=causal, mask=m, softcap=cap))
                ref = _sdpa64_ex(qf, kf, vf, scale, causal, m64, cap)
                assert np.abs(got - ref).max() < 2e-2 * np.abs(ref).max(), (causal, cap, kind)


# ------------------------------------------------------------------ C5 pieces
def test_rms_norm_reference_cases(oracle):
    g = GOLD["rms_norm_basic"]
    y = oracle.rms_norm_f32(np.array(g["x"], np.float32), g["eps"])
    exp = np.array(g["x"], np.float64) / np.sqrt(7.5 + 1e-5)
    assert np.abs(y - exp).max() < g["tol"] and np.abs(y - exp).max() < 1e-6
    g = GOLD["rms_norm_axis"]
    x = np.array(g["x"], np.float32)
    y = oracle.rms_norm_f32(x, g["eps"])
    exp = x / np.sqrt(np.array(g["row_mean_sq"])[:, None] + g["eps"])
    assert np.abs(y - exp).max() < 1e-6


def test_rms_norm_weight_bf16_vs_float64(oracle):
    x = synth.normal_bf16((17, 256), 5, 0)
    w = synth.to_bf16(1.0 + synth.normal((256,), 5, 1, sigma=0.1))
    y = synth.from_bf16(oracle.rms_norm_weight_bf16(x, w, 1e-6))
    xf = synth.from_bf16(x).astype(np.float64)
    ref = xf / np.sqrt((xf**2).mean(-1, keepdims=True) + 1e-6) * synth.from_bf16(w)
    assert np.all(np.abs(y - ref) <= np.abs(ref) * 2**-8 + 1e-6)


def test_rope_reference_cases(oracle):
    for key in ("rope_split", "rope_interleaved", "rope_rotation"):
        g = GOLD[key]
        y = oracle.rope_f32(np.array(g["x"], np.float32).reshape(1, 1, 4), np.array(g["cos"], np.float32),
                            np.array(g["sin"], np.float32), g["interleaved"])
        assert np.abs(y.ravel() - np.array(g["expected"])).max() < g["tol"], key


def test_rope_is_a_rotation(oracle):
    x = synth.normal((5, 7, 64), 5, 2)
    ang = synth.uniform((5, 7, 32), 5, 3, lo=-3.0, hi=3.0).astype(np.float64)
    for inter in (False, True):
        y = oracle.rope_f32(x, np.cos(ang), np.sin(ang), inter)
        if inter:
            z = x[..., 0::2].astype(np.float64) + 1j * x[..., 1::2]
            w = y[..., 0::2].astype(np.float64) + 1j * y[..., 1::2]
        else:
            z = x[..., :32].astype(np.float64) + 1j * x[..., 32:]
            w = y[..., :32].astype(np.float64) + 1j * y[..., 32:]
        assert np.abs(w - z * np.exp(1j * ang)).max() < 1e-5


def test_embedding_reference_cases(oracle):
    g = GOLD["embedding_basic"]
    w = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(oracle.embedding(w, np.array(g["indices"])), np.array(g["expected"], np.float32))
    g = GOLD["embedding_2d"]
    out = oracle.embedding(np.array(g["weight"], np.float32), np.array(g["indices"]))
    assert np.array_equal(out, np.array(g["expected"], np.float32))
    wb = synth.normal_bf16((50, 16), 5, 4)
    idx = synth.randint((3, 9), 5, 5, high=50)
    assert np.array_equal(oracle.embedding(wb, idx), wb[idx])


def test_silu_vs_float64(oracle):
    x = synth.uniform((4096,), 5, 6, lo=-12, hi=12)
    ref = x.astype(np.float64) / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.abs(oracle.silu_f32(x) - ref).max() < 2e-6
    g = synth.to_bf16(x)
    u = synth.normal_bf16((4096,), 5, 7)
    gf = synth.from_bf16(g).astype(np.float64)
    ref = gf / (1.0 + np.exp(-gf)) * synth.from_bf16(u)
    y = synth.from_bf16(oracle.silu_mul_bf16(g, u))
    assert np.all(np.abs(y - ref) <= np.abs(ref) * 2**-8 + 1e-6)


def test_decoder_block_composition_vs_float64(oracle):
    """The composed block equals a float64 evaluation of the same stage list (with the
    same bf16 roundings at stage outputs) within bf16 noise."""
    B, S, Hd, NH, F, V = 2, 24, 64, 4, 96, 40
    D = Hd // NH
    w = {
        "emb": synth.normal_bf16((V, Hd), 5, 10, 1.0),
        "w_an": synth.to_bf16(1.0 + synth.normal((Hd,), 5, 11, 0.1)),
        "w_fn": synth.to_bf16(1.0 + synth.normal((Hd,), 5, 12, 0.1)),
    }
    for i, (name, shp) in enumerate([("Wq", (Hd, Hd)), ("Wk", (Hd, Hd)), ("Wv", (Hd, Hd)), ("Wo", (Hd, Hd)),
                                     ("W1", (Hd, F)), ("W3", (Hd, F)), ("W2", (F, Hd))]):
        w[name] = synth.normal_bf16(shp, 5, 20 + i, 1.0 / np.sqrt(shp[0]))
    tok = synth.randint((B, S), 5, 30, high=V)
    inv = 10000.0 ** (-np.arange(0, D, 2) / D)
    ang = np.arange(S)[:, None] * inv[None, :]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    out = synth.from_bf16(oracle.decoder_block_bf16(tok, w, cos, sin, B, S, Hd, NH, F, 1e-6))

    f = {k: synth.from_bf16(v).astype(np.float64) for k, v in w.items()}
    r = lambda a: synth.from_bf16(synth.to_bf16(a.astype(np.float32))).astype(np.float64)  # noqa: E731
    h = f["emb"][tok.ravel()]
    rms = lambda x, g: r(x / np.sqrt((x**2).mean(-1, keepdims=True) + 1e-6) * g)  # noqa: E731
    xn = rms(h, f["w_an"])
    q, k, v = r(xn @ f["Wq"]), r(xn @ f["Wk"]), r(xn @ f["Wv"])

    def heads(t, rope):
        t = t.reshape(B, S, NH, D).transpose(0, 2, 1, 3)
        if rope:
            t1, t2 = t[..., : D // 2], t[..., D // 2:]
            t = np.concatenate([t1 * cos - t2 * sin, t1 * sin + t2 * cos], -1)
        return r(t)

    a = _sdpa64(heads(q, True), heads(k, True), heads(v, False), 1.0 / np.sqrt(D), True)
    a = r(a).transpose(0, 2, 1, 3).reshape(B * S, Hd)
    h2 = r(h + r(a @ f["Wo"]))
    xn2 = rms(h2, f["w_fn"])
    g1, g3 = r(xn2 @ f["W1"]), r(xn2 @ f["W3"])
    g = r(g1 / (1 + np.exp(-g1)) * g3)
    ref = r(h2 + r(g @ f["W2"]))
    assert np.abs(out - ref).max() < 3e-2 * np.abs(ref).max()


# ------------------------------------------------------------------ elementwise semantics tables
# orc_unary_f32 / orc_binary_f32 / orc_binary_i64 and their orc_map_* loops are the truth the
# renderer parity tests compare generated kernels with; they are pinned here against the known
# answers the reference holds, against float64 evaluation of the same function and, for the
# integer table, against brute force over small operands of both signs.
_UN = {"neg": 0, "abs": 1, "sqrt": 2, "rsqrt": 3, "reciprocal": 4, "exp": 5, "exp2": 6, "log": 7, "log2": 8,
       "sin": 9, "cos": 10, "tan": 11, "floor": 12, "ceil": 13, "trunc": 14, "round": 15, "erf": 16, "sign": 17,
       "square": 18}
_BF = {"add": 0, "sub": 1, "mul": 2, "fdiv": 3, "mod": 4, "max": 5, "pow": 6}
_BI = {"add": 0, "sub": 1, "mul": 2, "idiv": 3, "mod": 4, "max": 5, "and": 7, "or": 8, "xor": 9, "shl": 10, "shr": 11}


def _ulp_bound(ref64, ulps):
    """|error| allowed for a float32 result whose exact value is ref64."""
    return ulps * np.spacing(np.abs(ref64).astype(np.float32)).astype(np.float64)


def test_unary_table_vs_float64(oracle):
    import math

    pos = np.concatenate([synth.uniform((4000,), 91, 0, 1e-3, 60.0), np.float32([1, 4, 9, 0.25, 2, 1e-3])])
    sym = np.concatenate([synth.uniform((4000,), 91, 1, -30.0, 30.0), np.float32([0, -0.0, 1, -1, 2.5, -2.5, 0.5, -0.5, 1.5])])
    f64 = {
        "neg": (sym, lambda x: -x, 0), "abs": (sym, np.abs, 0), "sqrt": (pos, np.sqrt, 0.5),
        "rsqrt": (pos, lambda x: 1 / np.sqrt(x), 1.5), "reciprocal": (sym[sym != 0], lambda x: 1 / x, 0.5),
        "exp": (sym[np.abs(sym) < 20], np.exp, 2), "exp2": (sym[np.abs(sym) < 20], np.exp2, 2),
        "log": (pos, np.log, 2), "log2": (pos, np.log2, 2), "floor": (sym, np.floor, 0), "ceil": (sym, np.ceil, 0),
        "trunc": (sym, np.trunc, 0), "round": (sym, np.rint, 0), "sign": (sym, np.sign, 0),
        "square": (sym, lambda x: x * x, 0.5),
        "erf": (sym[np.abs(sym) < 4], np.vectorize(math.erf), 2), "tan": (sym[np.abs(sym) < 1.4], np.tan, 2),
    }
    for op, (x, fn, ulps) in f64.items():
        y = oracle.map_unary_f32(_UN[op], x).astype(np.float64)
        ref = fn(x.astype(np.float64))
        assert np.all(np.abs(y - ref) <= _ulp_bound(ref, ulps)), op
    # sin / cos: absolute bound near their zeros
    for op, fn in (("sin", np.sin), ("cos", np.cos)):
        y = oracle.map_unary_f32(_UN[op], sym).astype(np.float64)
        assert np.abs(y - fn(sym.astype(np.float64))).max() <= 2e-7, op
    # every op tag of the table is covered above
    assert set(f64) | {"sin", "cos"} == set(_UN)


def test_unary_table_distinguishing_values(oracle):
    """Values at which neighbouring ops of the table differ, so a swapped case label fails."""
    x = np.float32([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.7, -3.7])
    want = {
        "floor": [-3, -2, -1, 0, 1, 2, 3, -4], "ceil": [-2, -1, -0.0, 1, 2, 3, 4, -3],
        "trunc": [-2, -1, -0.0, 0, 1, 2, 3, -3], "round": [-2, -2, -0.0, 0, 2, 2, 4, -4],  # half to even
        "sign": [-1, -1, -1, 1, 1, 1, 1, -1], "neg": list(-x), "abs": list(np.abs(x)), "square": list(x * x),
    }
    for op, w in want.items():
        assert np.array_equal(oracle.map_unary_f32(_UN[op], x), np.float32(w)), op
    assert oracle.map_unary_f32(_UN["sign"], np.float32([0.0, -0.0])).tolist() == [0.0, 0.0]
    # exp / exp2 / log / log2 at points where the bases tell them apart
    assert abs(float(oracle.map_unary_f32(_UN["exp"], np.float32([1]))[0]) - np.e) < 3e-7
    assert oracle.map_unary_f32(_UN["exp2"], np.float32([3, 10, -1])).tolist() == [8.0, 1024.0, 0.5]
    assert oracle.map_unary_f32(_UN["log2"], np.float32([8, 0.25])).tolist() == [3.0, -2.0]
    assert abs(float(oracle.map_unary_f32(_UN["log"], np.float32([np.e]))[0]) - 1.0) < 2e-7
    assert oracle.map_unary_f32(_UN["sqrt"], np.float32([1, 4, 9])).tolist() == [1.0, 2.0, 3.0]
    assert oracle.map_unary_f32(_UN["rsqrt"], np.float32([1, 4, 16])).tolist() == [1.0, 0.5, 0.25]
    assert oracle.map_unary_f32(_UN["reciprocal"], np.float32([2, -4])).tolist() == [0.5, -0.25]
    # scalar entry point and the mapped loop agree
    assert oracle.lib.orc_unary_f32(_UN["square"], C.c_float(3.0)) == 9.0


def test_binary_f32_table(oracle):
    for c in GOLD["realize_binary"]["cases"]:  # tensor/src/test/unit/realize_binary.rs:16-270
        a, b = np.float32(c["a"]), np.float32(c["b"])
        y = oracle.map_binary_f32(_BF[c["op"]], a, b)
        want = np.float32(c["expected"]) if "expected" in c else {
            "add": np.add, "sub": np.subtract, "mul": np.multiply, "fdiv": np.divide}[c["op"]](a, b)
        assert np.abs(y - want).max() <= c["tol"], c["name"]
    a = synth.uniform((5000,), 92, 0, -8.0, 8.0)
    b = synth.uniform((5000,), 92, 1, 0.25, 4.0) * np.where(synth.uniform((5000,), 92, 2) > 0, 1, -1).astype(np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    for op, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("fdiv", np.divide)):
        # IEEE: the float32 result is the correctly rounded exact result
        assert np.array_equal(oracle.map_binary_f32(_BF[op], a, b), fn(a64, b64).astype(np.float32)), op
    assert np.array_equal(oracle.map_binary_f32(_BF["max"], a, b), np.maximum(a, b))
    # fmod: exact, sign of the dividend (C remainder, not Python's)
    assert np.array_equal(oracle.map_binary_f32(_BF["mod"], a, b), np.fmod(a64, b64).astype(np.float32))
    assert oracle.map_binary_f32(_BF["mod"], np.float32([-9, 9, 5.5]), np.float32([5, -5, 2])).tolist() == [-4.0, 4.0, 1.5]
    ap = np.abs(a) + np.float32(0.1)
    ref = np.power(ap.astype(np.float64), b64)
    assert np.all(np.abs(oracle.map_binary_f32(_BF["pow"], ap, b) - ref) <= _ulp_bound(ref, 2))
    # operand order: sub, fdiv, mod and pow are not commutative
    assert oracle.lib.orc_binary_f32(_BF["sub"], C.c_float(5), C.c_float(3)) == 2.0
    assert oracle.lib.orc_binary_f32(_BF["fdiv"], C.c_float(1), C.c_float(4)) == 0.25
    assert oracle.lib.orc_binary_f32(_BF["pow"], C.c_float(2), C.c_float(5)) == 32.0


def test_binary_integer_table_brute_force(oracle):
    """Brute force over operands of both signs against Python's unbounded integers, with C
    semantics written out: quotient truncated toward zero, remainder with the dividend's sign
    (ir/src/types.rs:625-646), arithmetic right shift, two's-complement wrap to 32 bits."""
    for c in GOLD["integer_div_mod_doc_examples"]["cases"]:
        got = oracle.map_binary_i32(_BI[c["op"]], np.int32([c["a"]]), np.int32([c["b"]]))
        assert int(got[0]) == c["expected"], c

    def wrap(v):
        return (v + 2**31) % 2**32 - 2**31

    def trunc_div(a, b):
        q = abs(a) // abs(b)
        return q if (a < 0) == (b < 0) else -q

    py = {"add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b, "idiv": trunc_div,
          "mod": lambda a, b: a - trunc_div(a, b) * b, "max": max, "and": lambda a, b: a & b,
          "or": lambda a, b: a | b, "xor": lambda a, b: a ^ b}
    vals = list(range(-20, 21)) + [2**31 - 1, -2**31 + 1, 123456789, -987654321, 65535, -65536]
    aa, bb = np.meshgrid(np.int32(vals), np.int32(vals), indexing="ij")
    aa, bb = aa.ravel(), bb.ravel()
    for op, fn in py.items():
        keep = bb != 0 if op in ("idiv", "mod") else np.ones(aa.shape, bool)
        a, b = aa[keep], bb[keep]
        got = oracle.map_binary_i32(_BI[op], a, b)
        want = np.array([wrap(fn(int(x), int(y))) for x, y in zip(a, b)], np.int64).astype(np.int32)
        assert np.array_equal(got, want), op
    sh = np.int32(list(range(0, 31)))
    for v in (1, 3, -1, -8, 1000, -123456, 2**30 + 5):
        a = np.full(sh.shape, v, np.int32)
        assert np.array_equal(oracle.map_binary_i32(_BI["shr"], a, sh), np.int32([v >> int(s) for s in sh])), v
    # left shifts are compared where the result fits (no signed overflow, which C leaves undefined)
    for v in (1, 3, 5, 1000):
        s = np.int32([k for k in range(0, 31) if abs(v) << k < 2**31])
        a = np.full(s.shape, v, np.int32)
        assert np.array_equal(oracle.map_binary_i32(_BI["shl"], a, s), np.int32([v << int(k) for k in s])), v
    assert set(py) | {"shl", "shr"} == set(_BI)
    # 64-bit scalar entry point: products beyond 32 bits are kept
    oracle.lib.orc_binary_i64.restype = C.c_longlong
    oracle.lib.orc_binary_i64.argtypes = [C.c_int, C.c_longlong, C.c_longlong]
    assert oracle.lib.orc_binary_i64(_BI["mul"], 3_000_000_000, 7) == 21_000_000_000
    assert oracle.lib.orc_binary_i64(_BI["idiv"], -21_000_000_001, 7) == -3_000_000_000
    assert oracle.lib.orc_binary_i64(_BI["mod"], -21_000_000_001, 7) == -1


def test_composed_activation_known_answers(oracle):
    """softplus / mish / softsign / sinh / cosh as the reference composes them from the table's
    ops (tensor/src/activation.rs:320-358, tensor/src/math.rs:252-266), against the values its
    own tests hold."""
    U = lambda op, x: oracle.map_unary_f32(_UN[op], x)
    B = lambda op, a, b: oracle.map_binary_f32(_BF[op], a, np.broadcast_to(np.float32(b), a.shape))

    def softplus(x, beta):
        s = B("mul", x, beta)
        m = B("max", s, 0.0)
        t = B("add", U("exp", B("sub", s, m)), U("exp", B("sub", np.zeros_like(x), m)))
        return B("mul", B("add", U("log", t), m), np.float32(1.0 / beta))

    def tanh(x):  # 2 * sigmoid(2x) - 1, sigmoid through exp2 (activation.rs:64-74)
        t = B("mul", x, 2.0)
        sig = U("reciprocal", B("add", U("exp2", B("mul", t, np.float32(-1.0 / np.log(2.0)))), 1.0))
        return B("sub", B("mul", sig, 2.0), 1.0)

    for c in GOLD["activation_values"]["cases"] + GOLD["math_values"]["cases"]:
        x = np.float32(c["x"])
        if c["name"] == "softplus":
            y = softplus(x, c["beta"])
        elif c["name"] == "mish":
            y = B("mul", x, tanh(softplus(x, 1.0)))
        elif c["name"] == "softsign":
            y = B("fdiv", x, B("add", U("abs", x), 1.0))
        else:
            ep, en = U("exp", x), U("exp", U("neg", x))
            y = B("fdiv", B("sub" if c["name"] == "sinh" else "add", ep, en), 2.0)
        assert np.abs(y - np.float32(c["expected"])).max() <= c["tol"], c
    g = GOLD["tanh_doc_values"]
    assert np.abs(tanh(np.float32(g["x"])) - np.float32(g["expected"])).max() <= g["tol"]


def test_add_bf16_definition(oracle):
    """y = bf16(float(a) + float(b)), round to nearest even: the float32 sum of two bf16 values
    is exact in float64, so rounding the float64 sum twice (to f32, then to bf16) is the
    definition; cases with ties and opposite signs included."""
    a = synth.normal_bf16((4096,), 93, 0)
    b = synth.normal_bf16((4096,), 93, 1)
    s32 = (synth.from_bf16(a).astype(np.float64) + synth.from_bf16(b).astype(np.float64)).astype(np.float32)
    assert np.array_equal(oracle.add_bf16(a, b), synth.to_bf16(s32))
    one, eps = synth.to_bf16(np.float32([1.0])), synth.to_bf16(np.float32([2.0 ** -8]))
    # 1 + 2^-8 lies halfway between 1 and the next bf16 (1 + 2^-7): ties go to the even mantissa
    assert synth.from_bf16(oracle.add_bf16(one, eps))[0] == 1.0
    x = synth.to_bf16(np.float32([1.0 + 2.0 ** -7]))
    assert synth.from_bf16(oracle.add_bf16(x, eps))[0] == np.float32(1.0 + 2.0 ** -6)
    assert synth.from_bf16(oracle.add_bf16(x, synth.to_bf16(np.float32([-1.0]))))[0] == np.float32(2.0 ** -7)


def test_bf16_conversions_round_to_nearest_even_over_every_code(oracle):
    """orc_bf16_to_f32 over all 65536 codes is the code shifted into the upper half of a
    float32; orc_f32_to_bf16 is pinned without restating its bit trick: for every finite bf16
    value v with successor w, everything strictly below the midpoint rounds to v, everything
    above to w, and the midpoint itself to whichever of the two has an even mantissa (computed
    in float64, where v, w and their midpoint are exact); NaN stays NaN, the largest float32
    values round to infinity."""
    codes = np.arange(65536, dtype=np.uint16)
    f = np.empty(65536, np.float32)
    oracle.lib.orc_bf16_to_f32(codes.ctypes.data_as(C.c_void_p), f.ctypes.data_as(C.c_void_p), C.c_long(65536))
    assert np.array_equal(f.view(np.uint32), codes.astype(np.uint32) << 16)

    def to_bf16(x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.uint16)
        oracle.lib.orc_f32_to_bf16(x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), C.c_long(x.size))
        return out

    assert np.array_equal(to_bf16(f[np.isfinite(f)]), codes[np.isfinite(f)])        # exact values keep their code
    pos = codes[(codes < 0x7f7f)]                                                    # positive finite, successor finite
    v, w = f[pos].astype(np.float64), f[pos + 1].astype(np.float64)
    mid = (v + w) / 2                                                                # exact: one more mantissa bit
    below = np.nextafter(mid.astype(np.float32), np.float32(0)).astype(np.float32)
    above = np.nextafter(mid.astype(np.float32), np.float32(np.inf)).astype(np.float32)
    assert np.array_equal(mid.astype(np.float32).astype(np.float64), mid)
    assert np.array_equal(to_bf16(below), pos) and np.array_equal(to_bf16(above), pos + 1)
    even = np.where(pos % 2 == 0, pos, pos + 1)
    assert np.array_equal(to_bf16(mid.astype(np.float32)), even)
    assert np.array_equal(to_bf16(-mid.astype(np.float32)), even | 0x8000)           # sign symmetric
    big = np.float32([3.4e38, -3.4e38, np.inf, -np.inf])
    assert np.array_equal(to_bf16(big), np.uint16([0x7f80, 0xff80, 0x7f80, 0xff80]))
    nan = to_bf16(np.float32([np.nan]))[0]
    assert (nan & 0x7f80) == 0x7f80 and (nan & 0x7f) != 0


def test_f16_conversions_over_every_code_and_gemm_f16_by_definition(oracle):
    """orc_f16_to_f32 against numpy's IEEE half over all 65536 codes (subnormals, infinities, NaN);
    orc_f32_to_f16 against numpy's float32 -> float16 rounding on every midpoint between neighbouring
    halves, its two float32 neighbours, the overflow boundary 65520 and random values; orc_gemm_f16
    against the float64 product of the same f16 inputs and against cases with exact answers."""
    codes = np.arange(65536, dtype=np.uint16)
    f = np.empty(65536, np.float32)
    oracle.lib.orc_f16_to_f32(codes.ctypes.data_as(C.c_void_p), f.ctypes.data_as(C.c_void_p), C.c_long(65536))
    want = codes.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(f[np.isnan(want)]).all()

    def to_f16(x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.uint16)
        oracle.lib.orc_f32_to_f16(x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), C.c_long(x.size))
        return out

    fin = np.isfinite(want)
    assert np.array_equal(to_f16(want[fin]), codes[fin])
    pos = codes[codes < 0x7bff]
    v, w = want[pos].astype(np.float64), want[pos + 1].astype(np.float64)
    mid = ((v + w) / 2).astype(np.float32)
    trial = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)), -mid,
                            np.float32([65504.0, 65519.99, 65520.0, 65536.0, 1e9, -65520.0, np.inf, 0.0, -0.0, 1e-10, 2.0 ** -25, 2.0 ** -24 * 1.5]),
                            synth.normal((20000,), 97, 0) * np.float32(100.0), synth.normal((20000,), 97, 1) * np.float32(1e-5)])
    with np.errstate(over="ignore"):
        assert np.array_equal(to_f16(trial), trial.astype(np.float16).view(np.uint16))
    nan = to_f16(np.float32([np.nan]))[0]
    assert (nan & 0x7c00) == 0x7c00 and (nan & 0x3ff) != 0
    M, N, K = 37, 29, 200
    a = synth.normal((M, K), 97, 2).astype(np.float16)
    b = synth.normal((K, N), 97, 3).astype(np.float16)
    got = oracle.gemm_f16(a, b).astype(np.float64)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(got - ref).max() <= 1.5e-3 * np.abs(ref).max()           # one f16 rounding (2^-11) + f32 accumulation
    eye = np.eye(K, dtype=np.float16)
    assert np.array_equal(oracle.gemm_f16(a, eye), a)                       # identity: exact
    ones = np.ones((K, N), np.float16)
    small = (synth.uniform((M, K), 97, 4) * 8).astype(np.int32).astype(np.float16)   # small integers: sums exact
    assert np.array_equal(oracle.gemm_f16(small, ones).astype(np.float64), small.astype(np.float64).sum(1, keepdims=True).repeat(N, 1))
    # transposed operand order matters: a dropped transpose or a swapped index fails here
    assert not np.allclose(oracle.gemm_f16(a[:29, :29], b[:29, :29].T.copy()).astype(np.float64), ref[:29, :29], atol=1e-2)


def test_heads_to_tokens_and_rope_heads_layout(oracle):
    """Index checks with distinct values per position: [B,H,S,D] -> [B*S, H*D] and the
    token-major -> head-major move of orc_rope_heads_bf16 (apply=0: a pure permutation;
    apply=1: the split-half rotation of orc_rope_f32 on every head)."""
    Bn, S, H, D = 2, 5, 3, 8
    x = np.arange(Bn * H * S * D, dtype=np.uint16).reshape(Bn, H, S, D)
    y = np.empty((Bn * S, H * D), np.uint16)
    oracle.lib.orc_heads_to_tokens_u16(x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p), Bn, S, H, D)
    assert np.array_equal(y, x.transpose(0, 2, 1, 3).reshape(Bn * S, H * D))
    tok = synth.normal_bf16((Bn * S, H * D), 94, 0)
    ang = synth.uniform((S, D // 2), 94, 1, -3.0, 3.0)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    moved = oracle.rope_heads_bf16(tok, cos, sin, Bn, S, H, D, apply=False)
    assert np.array_equal(moved, tok.reshape(Bn, S, H, D).transpose(0, 2, 1, 3))
    rot = oracle.rope_heads_bf16(tok, cos, sin, Bn, S, H, D, apply=True)
    xf = synth.from_bf16(moved).astype(np.float64)
    c64, s64 = cos.astype(np.float64), sin.astype(np.float64)
    lo, hi = xf[..., : D // 2], xf[..., D // 2:]
    ref = np.concatenate([lo * c64 - hi * s64, lo * s64 + hi * c64], -1)
    got = synth.from_bf16(rot).astype(np.float64)
    assert np.abs(got - ref).max() <= 2.0 ** -8 * np.abs(ref).max() + 1e-6


def test_fp8_decode_all_codes(oracle):
    """Every one of the 256 codes of both 8-bit floats.  E5M2 is the top byte of an IEEE half, so
    numpy's float16 decodes it independently; E4M3 (OCP: bias 7, no infinity, S.1111.111 = NaN)
    against its closed form written per field; both against the range and field widths the
    reference records for them."""
    codes = np.arange(256, dtype=np.uint8)
    fmt = GOLD["fp8_formats"]
    e5 = oracle.fp8_to_f32(1, codes)
    half = (codes.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(e5), np.isnan(half)) and np.array_equal(e5[~np.isnan(e5)], half[~np.isnan(half)])
    fin = e5[np.isfinite(e5)]
    assert fin.max() == fmt["e5m2"]["max"] and fin.min() == fmt["e5m2"]["min"]
    e4 = oracle.fp8_to_f32(0, codes)
    eb, mb = fmt["e4m3"]["exponent_bits"], fmt["e4m3"]["mantissa_bits"]
    assert (eb, mb) == (4, 3) and 1 + eb + mb == 8
    want = []
    for c in range(256):
        s, e, m = c >> 7, (c >> mb) & (2 ** eb - 1), c & (2 ** mb - 1)
        if e == 2 ** eb - 1 and m == 2 ** mb - 1:
            v = float("nan")
        elif e == 0:
            v = m / 2 ** mb * 2.0 ** (1 - 7)
        else:
            v = (1 + m / 2 ** mb) * 2.0 ** (e - 7)
        want.append(-v if s else v)
    want = np.float32(want)
    assert np.isnan(e4[0x7F]) and np.isnan(e4[0xFF]) and np.isnan(e4).sum() == 2 and not np.isinf(e4).any()
    ok = ~np.isnan(want)
    assert np.array_equal(e4[ok], want[ok])
    assert np.nanmax(e4) == fmt["e4m3"]["max"] and np.nanmin(e4) == fmt["e4m3"]["min"]
    # landmarks a shifted bias or a swapped field width would move
    assert e4[0x38] == 1.0 and e4[0x40] == 2.0 and e4[0x30] == 0.5 and e4[0x01] == 2.0 ** -9 and e4[0x08] == 2.0 ** -6 and e4[0x7E] == 448.0
    assert e5[0x3C] == 1.0 and e5[0x40] == 2.0 and e5[0x01] == 2.0 ** -16 and e5[0x7B] == 57344.0 and np.isinf(e5[0x7C])
    # magnitudes grow with the code within a sign
    assert np.all(np.diff(e4[:0x7F]) > 0) and np.all(np.diff(e5[:0x7D]) > 0)


@pytest.mark.parametrize("kind", [0, 1])
def test_fp8_matmul_vs_float64(oracle, kind):
    rng = np.random.default_rng(95 + kind)
    M, N, K = 33, 20, 96
    # finite codes of moderate magnitude
    a = rng.integers(0x10, 0x58, (M, K)).astype(np.uint8) | (rng.integers(0, 2, (M, K)).astype(np.uint8) << 7)
    b = rng.integers(0x10, 0x58, (K, N)).astype(np.uint8) | (rng.integers(0, 2, (K, N)).astype(np.uint8) << 7)
    c = oracle.matmul_fp8_f32(kind, a, b)
    af, bf = oracle.fp8_to_f32(kind, a).astype(np.float64), oracle.fp8_to_f32(kind, b).astype(np.float64)
    ref = af @ bf
    assert np.abs(c - ref).max() <= 1e-5 * (np.abs(af) @ np.abs(bf)).max()
    eye = np.zeros((K, K), np.uint8)
    eye[np.arange(K), np.arange(K)] = 0x38 if kind == 0 else 0x3C        # 1.0
    assert np.array_equal(oracle.matmul_fp8_f32(kind, a, eye), oracle.fp8_to_f32(kind, a))
