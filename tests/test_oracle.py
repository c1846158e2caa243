"""Pins the CPU oracle (oracle/morok_cpu_oracle.c) before anything is compared with it:
against the known answers held by the reference's own tests (tests/golden/
reference_known_answers.json) and against what the mathematics fixes (float64 closed forms,
invariants, special cases).  Runs without a GPU."""
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
