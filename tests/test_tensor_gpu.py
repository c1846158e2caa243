"""Lazy tensor API on the GPU: the reference's own tensor tests restated through the C ABI
(tensor/src/test/unit/matmul.rs, transformer.rs, fusion.rs, book_examples.rs), every result
also checked against the CPU oracle.  Both lowering modes are covered: generated kernels only
(fusion off) and the hand-written kernels (fusion on)."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


@pytest.fixture()
def T(dev):
    from morok_amd import tensor

    yield tensor
    tensor.set_fusion(True)


@pytest.fixture(params=[False, True], ids=["generated", "fused"])
def fusion(request, T):
    T.set_fusion(request.param)
    return request.param


def f32(a):
    return np.asarray(a, dtype=np.float32)


# ---------------------------------------------------------------- creation / extraction
def test_roundtrip_and_size_check(T):
    from morok_amd import MorokHipError, uop

    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = T.Tensor.from_numpy(x)
    assert t.shape == (2, 3, 4) and t.dtype == uop.F32
    np.testing.assert_array_equal(t.to_numpy(), x)
    with pytest.raises(MorokHipError) as e:  # data.rs:81-96
        T.Tensor.from_bytes(b"\0" * 10, (3,), uop.F32)
    assert "data length 10 != expected 12" in str(e.value)
    assert e.value.code == 1


def test_movement_ops_are_index_arithmetic(T):
    x = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    t = T.Tensor.from_numpy(x)
    y = t.try_permute([2, 0, 1]).try_reshape([4, 6]).try_shrink([(1, 3), (2, 5)]).try_add(1.0)
    np.testing.assert_array_equal(y.to_numpy(), x.transpose(2, 0, 1).reshape(4, 6)[1:3, 2:5] + 1)
    assert len(y.kernels()) == 1  # one elementwise kernel, no copies for the views
    e = T.Tensor.from_numpy(f32([[1], [2]])).try_expand([2, 3]).try_mul(T.Tensor.from_numpy(f32([10, 20, 30])))
    np.testing.assert_array_equal(e.to_numpy(), f32([[10, 20, 30], [20, 40, 60]]))
    c = T.Tensor.cat([t, t.try_mul(2.0)], 1)
    np.testing.assert_array_equal(c.to_numpy(), np.concatenate([x, 2 * x], 1))


def test_elementwise_int_and_promotion(T):
    from morok_amd import uop

    a = T.Tensor.from_numpy(np.arange(-5, 5, dtype=np.int32))
    b = T.Tensor.from_numpy(np.full(10, 3, dtype=np.int32))
    np.testing.assert_array_equal(a.binary("mul", b).binary("add", b).to_numpy(), np.arange(-5, 5) * 3 + 3)
    m = a.binary("lt", 0)
    assert m.dtype == uop.BOOL
    np.testing.assert_array_equal(m.to_numpy(), np.arange(-5, 5) < 0)
    f = a.try_add(T.Tensor.from_numpy(np.full(10, 0.5, dtype=np.float32)))
    assert f.dtype == uop.F32
    np.testing.assert_array_equal(f.to_numpy(), np.arange(-5, 5) + np.float32(0.5))
    i64 = T.Tensor.from_numpy(np.array([2**40, -7], dtype=np.int64)).binary("add", T.Tensor.from_numpy(np.array([1, 1], dtype=np.int64)))
    np.testing.assert_array_equal(i64.to_numpy(), np.array([2**40 + 1, -6], dtype=np.int64))


# ---------------------------------------------------------------- matmul (matmul.rs)
def test_matmul_known_answers(T, fusion):
    for key in ("matmul_2x2", "matmul_3x3"):
        g = GOLD[key]
        c = T.Tensor.from_numpy(f32(g["a"])).matmul(T.Tensor.from_numpy(f32(g["b"])))
        np.testing.assert_allclose(c.to_numpy(), f32(g["expected"]), atol=g["tol"])


@pytest.mark.parametrize("n,tol", [(128, 0.5), (256, 1.0), (500, 1.5)])
def test_matmul_square_closed_form(T, fusion, oracle, n, tol):
    x = np.arange(n * n, dtype=np.int64)
    a = ((x % 31) * 0.05 - 0.8).astype(np.float32).reshape(n, n)
    b = ((x % 37) * 0.04 - 0.7).astype(np.float32).reshape(n, n)
    c = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b))
    got = c.to_numpy()
    assert len(c.kernels()) == 1  # fusion.rs:28-33
    ref = oracle.matmul_f32(a, b)
    assert np.abs(got - ref).max() < tol  # the reference's own tolerance (matmul.rs:669-677)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())


def test_matmul_config1_1024_cubed(T, oracle):
    """The first benchmark configuration itself: A[1024x1024] @ B[1024x1024], entries uniform(-1, 1)
    from seed 1, through Tensor::matmul (one generated kernel) against the CPU oracle on the same
    inputs; also the reference's closed-form generators at this size (matmul.rs:669-677)."""
    from morok_amd import synth

    n = 1024
    a, b = synth.uniform((n, n), 1, 0), synth.uniform((n, n), 1, 1)
    c = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b))
    got = c.to_numpy()
    assert c.kernels() == ["r_1024_1024_1024"]
    ref = oracle.matmul_f32(a, b)
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()  # f32 reduction tolerance
    x = np.arange(n * n, dtype=np.int64)
    a2 = ((x % 31) * 0.05 - 0.8).astype(np.float32).reshape(n, n)
    b2 = ((x % 37) * 0.04 - 0.7).astype(np.float32).reshape(n, n)
    got2 = T.Tensor.from_numpy(a2).matmul(T.Tensor.from_numpy(b2)).to_numpy()
    assert np.abs(got2 - oracle.matmul_f32(a2, b2)).max() < 3.0  # the reference's tolerance at 1024


def test_matmul_nonsquare_and_batched(T, fusion, oracle):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((64, 512), dtype=np.float32)
    b = rng.standard_normal((512, 64), dtype=np.float32)
    got = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b)).to_numpy()
    np.testing.assert_allclose(got, oracle.matmul_f32(a, b), rtol=1e-4, atol=1e-3)
    ab = rng.standard_normal((3, 5, 7), dtype=np.float32)
    bb = rng.standard_normal((3, 7, 4), dtype=np.float32)
    got = T.Tensor.from_numpy(ab).matmul(T.Tensor.from_numpy(bb)).to_numpy()
    np.testing.assert_allclose(got, np.stack([oracle.matmul_f32(ab[i], bb[i]) for i in range(3)]), rtol=1e-4, atol=1e-5)


def test_matmul_vector_operands(T, fusion):
    """tensor/src/test/unit/matmul.rs:176-235: 1-D @ 1-D is a scalar (70 for the reference's
    vectors), [4] @ [4, 3] -> [3], [3, 4] @ [4] -> [3]; larger random cases against numpy."""
    a = np.array([1, 2, 3, 4, 5], np.float32)
    b = np.array([2, 3, 4, 5, 6], np.float32)
    d = T.Tensor.from_numpy(a).dot(T.Tensor.from_numpy(b))
    assert d.shape == () and abs(float(d.to_numpy().reshape(-1)[0]) - 70.0) < 1e-5
    v = np.array([1, 2, 3, 4], np.float32)
    m = np.arange(1, 13, dtype=np.float32).reshape(4, 3)
    vm = T.Tensor.from_numpy(v).dot(T.Tensor.from_numpy(m))
    assert vm.shape == (3,)
    np.testing.assert_allclose(vm.to_numpy(), v @ m, atol=1e-5)
    m2 = np.arange(1, 13, dtype=np.float32).reshape(3, 4)
    mv = T.Tensor.from_numpy(m2).dot(T.Tensor.from_numpy(v))
    assert mv.shape == (3,)
    np.testing.assert_allclose(mv.to_numpy(), m2 @ v, atol=1e-5)
    rng = np.random.default_rng(81)
    x, w, y = rng.standard_normal(300).astype(np.float32), rng.standard_normal((300, 70)).astype(np.float32), \
        rng.standard_normal((5, 40, 300)).astype(np.float32)
    for lhs, rhs in ((x, w), (w.T.copy(), x), (y, x), (x, x)):
        got = T.Tensor.from_numpy(lhs).matmul(T.Tensor.from_numpy(rhs)).to_numpy()
        want = lhs.astype(np.float64) @ rhs.astype(np.float64)
        np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-4, atol=1e-4)


def test_matmul_dtype_options(T, fusion):
    """matmul.rs tests 417-435: int32 @ float32 promotes to float32; matmul_with().dtype(f64)
    accumulates the f32 products in float64 and returns float64."""
    from morok_amd import uop

    ai = np.array([[1, 2], [3, 4]], np.int32)
    bf = np.array([[5.0, 6.0], [7.0, 8.0]], np.float32)
    c = T.Tensor.from_numpy(ai).dot(T.Tensor.from_numpy(bf))
    assert c.dtype == uop.F32
    np.testing.assert_allclose(c.to_numpy(), ai @ bf)
    rng = np.random.default_rng(82)
    a = (rng.standard_normal((8, 4096)) * 1e3).astype(np.float32)
    b = rng.standard_normal((4096, 8)).astype(np.float32)
    c64 = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), dtype=uop.F64)
    assert c64.dtype == uop.F64
    got = c64.to_numpy()
    # the reference casts the f32 products, not the operands (matmul.rs:107-109): each product is
    # rounded to f32, the sum of 4096 of them is exact to f64 rounding
    want = (a[:, :, None] * b[None, :, :]).astype(np.float64).sum(axis=1)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-7)


def test_linear_and_gemm(T, fusion):
    """matmul.rs:513-566 (linear: bias, no bias, batched, 1-D weight) and gemm (alpha, beta,
    transposes, C), values against numpy."""
    x = np.array([[1.0, 2.0, 3.0]], np.float32)
    w = np.array([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], np.float32)
    bias = np.array([0.1, 0.2], np.float32)
    r = T.Tensor.from_numpy(x).linear(T.Tensor.from_numpy(w), T.Tensor.from_numpy(bias))
    assert r.shape == (1, 2)
    np.testing.assert_allclose(r.to_numpy(), x @ w.T + bias, rtol=1e-6)
    r = T.Tensor.from_numpy(x).linear(T.Tensor.from_numpy(w))
    assert r.shape == (1, 2)
    np.testing.assert_allclose(r.to_numpy(), x @ w.T, rtol=1e-6)
    r = T.Tensor.from_numpy(np.ones((4, 3), np.float32)).linear(T.Tensor.from_numpy(np.ones((2, 3), np.float32)))
    assert r.shape == (4, 2) and np.all(r.to_numpy() == 3.0)
    r = T.Tensor.from_numpy(np.array([1, 2, 3], np.float32)).linear(T.Tensor.from_numpy(np.array([2, 3, 4], np.float32)))
    assert r.shape == (3,) and np.all(r.to_numpy() == [2, 6, 12])
    rng = np.random.default_rng(83)
    a, b, c = (rng.standard_normal(sh).astype(np.float32) for sh in ((64, 48), (32, 48), (64, 32)))
    g = T.Tensor.from_numpy(a).gemm(T.Tensor.from_numpy(b), alpha=0.5, beta=2.0, trans_b=True, c=T.Tensor.from_numpy(c))
    np.testing.assert_allclose(g.to_numpy(), 0.5 * (a @ b.T) + 2.0 * c, rtol=1e-4, atol=1e-4)
    g = T.Tensor.from_numpy(a.T.copy()).gemm(T.Tensor.from_numpy(b.T.copy()), trans_a=True)
    np.testing.assert_allclose(g.to_numpy(), a @ b.T, rtol=1e-4, atol=1e-4)


def test_matmul_shape_error(T):
    from morok_amd import MorokHipError

    with pytest.raises(MorokHipError):
        T.Tensor.from_numpy(np.zeros((2, 3), np.float32)).matmul(T.Tensor.from_numpy(np.zeros((4, 2), np.float32)))


def test_matmul_bf16(T, fusion, oracle):
    from morok_amd import synth, uop

    rng = np.random.default_rng(7)
    M, N, K = (256, 256, 128) if fusion else (48, 40, 64)
    a = synth.to_bf16(rng.standard_normal((M, K), dtype=np.float32))
    b = synth.to_bf16(rng.standard_normal((K, N), dtype=np.float32))
    c = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(b, uop.BF16))
    assert c.dtype == uop.BF16
    got = synth.from_bf16(c.to_numpy())
    ref = synth.from_bf16(oracle.gemm_bf16(a, b))
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    if fusion:
        assert c.kernels() == ["gemm_bf16_tile256"] or c.kernels()[0].startswith("gemm_bf16")


@pytest.mark.parametrize("ashape,wshape", [((3, 100, 64), (64, 40)), ((2, 3, 128, 64), (2, 3, 64, 72)),
                                           ((5, 37, 128), (5, 128, 8)), ((2, 2, 50, 192), (192, 264))])
def test_matmul_bf16_leading_axes(T, fusion, oracle, ashape, wshape):
    """[..., M, K] x [K, N] (one product over the flattened leading axes) and [..., M, K] x
    [..., K, N] with equal leading axes (that many products, one launch of the hand-written
    kernel); generated and hand-written paths against the per-matrix oracle."""
    from morok_amd import synth, uop

    rng = np.random.default_rng(9)
    a = synth.to_bf16(rng.standard_normal(ashape, dtype=np.float32))
    w = synth.to_bf16(rng.standard_normal(wshape, dtype=np.float32))
    c = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(w, uop.BF16))
    got = synth.from_bf16(c.to_numpy())
    M, K, N = ashape[-2], ashape[-1], wshape[-1]
    a2 = a.reshape(-1, M, K)
    w2 = w.reshape(-1, K, N) if len(wshape) > 2 else np.broadcast_to(w, (a2.shape[0], K, N))
    ref = np.stack([synth.from_bf16(oracle.gemm_bf16(np.ascontiguousarray(a2[i]), np.ascontiguousarray(w2[i])))
                    for i in range(a2.shape[0])]).reshape(got.shape)
    assert got.shape == tuple(ashape[:-1]) + (N,)
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    if fusion:
        names = c.kernels()
        assert len(names) == 1 and names[0].startswith("gemm_bf16")
        assert names[0].endswith("_x%d" % a2.shape[0]) == (len(wshape) > 2)


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("shape", [(4, 8), (3, 1000), (2, 5, 257)])
def test_softmax(T, fusion, oracle, shape):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    s = T.Tensor.from_numpy(x).softmax(-1)
    got = s.to_numpy()
    assert len(s.kernels()) == (1 if fusion else 3)  # fusion.rs:83-88: max, sum, divide
    ref = oracle.softmax_f32(x.reshape(-1, shape[-1])).reshape(shape)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(got.sum(-1), 1.0, atol=GOLD["softmax_invariants"]["row_sum_tol"])
    assert (got > 0).all() and (got <= 1).all()


@pytest.mark.parametrize("axis", [-1, 0, 1])
def test_log_softmax_and_logsumexp(T, fusion, axis):
    """activation.rs:117-157 against float64 closed forms, including rows whose naive
    exp would overflow."""
    rng = np.random.default_rng(91)
    x = (rng.standard_normal((6, 50, 33)) * 30).astype(np.float32)
    x[0, 0] += 500.0
    x64 = x.astype(np.float64)
    m = x64.max(axis, keepdims=True)
    lse = m + np.log(np.exp(x64 - m).sum(axis, keepdims=True))
    got = T.Tensor.from_numpy(x).log_softmax(axis).to_numpy()
    np.testing.assert_allclose(got, x64 - lse, rtol=1e-5, atol=1e-4)
    got = T.Tensor.from_numpy(x).logsumexp(axis).to_numpy()
    assert got.shape == np.squeeze(lse, axis).shape
    np.testing.assert_allclose(got, np.squeeze(lse, axis), rtol=1e-5, atol=1e-4)
    assert np.allclose(np.exp(T.Tensor.from_numpy(x).log_softmax(axis).to_numpy().astype(np.float64)).sum(axis), 1.0, atol=1e-4)


def test_softmax_inner_axis(T, oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((6, 33, 5)).astype(np.float32)
    got = T.Tensor.from_numpy(x).softmax(1).to_numpy()
    ref = oracle.softmax_f32(np.ascontiguousarray(x.transpose(0, 2, 1)).reshape(-1, 33)).reshape(6, 5, 33).transpose(0, 2, 1)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-7)


# ---------------------------------------------------------------- reductions
def test_reductions(T):
    rng = np.random.default_rng(13)
    x = rng.standard_normal((7, 300, 9)).astype(np.float32)
    t = T.Tensor.from_numpy(x)
    np.testing.assert_allclose(t.sum(1).to_numpy(), x.astype(np.float64).sum(1), rtol=1e-4, atol=1e-4)
    np.testing.assert_array_equal(t.max(1).to_numpy(), x.max(1))
    np.testing.assert_allclose(t.sum([0, 2]).to_numpy(), x.astype(np.float64).sum((0, 2)), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(t.mean([2], keepdim=True).to_numpy(), x.mean(2, keepdims=True), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(t.sum([0, 1, 2]).to_numpy(), x.astype(np.float64).sum(), rtol=1e-4, atol=1e-3)
    i = np.arange(1000, dtype=np.int32).reshape(10, 100)
    np.testing.assert_array_equal(T.Tensor.from_numpy(i).sum(1).to_numpy(), i.sum(1))
    np.testing.assert_array_equal(T.Tensor.from_numpy(i).max(0).to_numpy(), i.max(0))


def test_sum_of_bf16_accumulates_in_f32(T):
    from morok_amd import synth, uop

    x = synth.to_bf16(np.full((4, 4096), 1.0 / 256, dtype=np.float32))
    s = T.Tensor.from_numpy(x, uop.BF16).sum(1)
    assert s.dtype == uop.BF16  # cast back after the promoted accumulation (reduce.rs:665-691)
    np.testing.assert_array_equal(synth.from_bf16(s.to_numpy()), np.full(4, 16.0, np.float32))


# ---------------------------------------------------------------- transformer.rs
def test_rms_norm(T):
    g = GOLD["rms_norm_basic"]
    x = f32(g["x"])
    got = T.Tensor.from_numpy(x).rms_norm(-1, g["eps"]).to_numpy()
    np.testing.assert_allclose(got, x / np.sqrt(7.5 + 1e-5), atol=g["tol"])
    g = GOLD["rms_norm_axis"]
    x = f32(g["x"])
    got = T.Tensor.from_numpy(x).rms_norm(-1, g["eps"]).to_numpy()
    np.testing.assert_allclose(got, x / np.sqrt(f32(g["row_mean_sq"])[:, None] + g["eps"]), atol=g["tol"])


def test_rms_norm_vs_oracle(T, oracle):
    rng = np.random.default_rng(17)
    x = rng.standard_normal((33, 4096)).astype(np.float32)
    got = T.Tensor.from_numpy(x).rms_norm(-1, 1e-6).to_numpy()
    np.testing.assert_allclose(got, oracle.rms_norm_f32(x, 1e-6), rtol=1e-5, atol=1e-6)


def test_embedding(T):
    g = GOLD["embedding_basic"]
    w = T.Tensor.from_numpy(np.arange(12, dtype=np.float32).reshape(3, 4))
    got = w.embedding(T.Tensor.from_numpy(np.array(g["indices"], dtype=np.int32))).to_numpy()
    np.testing.assert_array_equal(got, f32(g["expected"]))
    g = GOLD["embedding_2d"]
    got = T.Tensor.from_numpy(f32(g["weight"])).embedding(T.Tensor.from_numpy(np.array(g["indices"], dtype=np.int32))).to_numpy()
    np.testing.assert_array_equal(got, f32(g["expected"]))


@pytest.mark.parametrize("key", ["rope_split", "rope_interleaved", "rope_rotation"])
def test_rope_known_answers(T, key):
    g = GOLD[key]
    x = T.Tensor.from_numpy(f32(g["x"]).reshape(1, 1, 1, 4))
    cos = T.Tensor.from_numpy(f32(g["cos"]).reshape(1, 1, 1, 2))
    sin = T.Tensor.from_numpy(f32(g["sin"]).reshape(1, 1, 1, 2))
    got = x.apply_rotary_emb(cos, sin, g["interleaved"]).to_numpy().reshape(-1)
    np.testing.assert_allclose(got, f32(g["expected"]), atol=g["tol"])


@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_vs_oracle(T, oracle, interleaved):
    rng = np.random.default_rng(19)
    B, H, S, D = 2, 3, 17, 64
    x = rng.standard_normal((B, H, S, D)).astype(np.float32)
    ang = rng.uniform(0, 6.28, (S, D // 2)).astype(np.float32)
    cos, sin = np.cos(ang), np.sin(ang)
    got = T.Tensor.from_numpy(x).apply_rotary_emb(T.Tensor.from_numpy(cos.reshape(1, 1, S, D // 2)),
                                                  T.Tensor.from_numpy(sin.reshape(1, 1, S, D // 2)), interleaved).to_numpy()
    ref = oracle.rope_f32(x, cos, sin, interleaved)
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_sdpa_causal_row0(T, fusion):
    g = GOLD["sdpa_causal_row0"]
    q = T.Tensor.from_numpy(f32(g["q"]).reshape(1, 1, 3, 2))
    v = T.Tensor.from_numpy(f32(g["v"]).reshape(1, 1, 3, 2))
    out = q.scaled_dot_product_attention(q, v, is_causal=True).to_numpy()
    assert out.shape == (1, 1, 3, 2)
    np.testing.assert_allclose(out[0, 0, 0], f32(g["expected_row0"]), atol=g["tol"])


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_f32_vs_oracle(T, fusion, oracle, causal):
    rng = np.random.default_rng(23)
    B, H, S, D = 2, 2, 40, 16
    q, k, v = (rng.standard_normal((B, H, S, D)).astype(np.float32) for _ in range(3))
    out = T.Tensor.from_numpy(q).scaled_dot_product_attention(T.Tensor.from_numpy(k), T.Tensor.from_numpy(v),
                                                              is_causal=causal).to_numpy()
    ref = oracle.sdpa_f32(q, k, v, 1 / np.sqrt(D), causal)
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5)


def _np_sdpa(q, k, v, scale, causal=False, mask=None, softcap=None):
    s = np.einsum("bhqd,bhkd->bhqk", q.astype(np.float64), k.astype(np.float64)) * scale
    if causal:
        s = np.where(np.tril(np.ones(s.shape[-2:], bool)), s, -np.inf)
    if mask is not None:
        s = s + (np.where(mask, 0.0, -np.inf) if mask.dtype == np.bool_ else mask.astype(np.float64))
    if softcap:
        s = np.tanh(s / softcap) * softcap
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", p, v.astype(np.float64))


def test_tanh(T, fusion):
    """tanh = 2 * sigmoid(2x) - 1 (activation.rs:64-74); the reference's doc values."""
    x = np.array([-2.0, -1.0, 0.0, 1.0, 2.0, 9.0, -30.0], np.float32)
    got = T.Tensor.from_numpy(x).tanh().to_numpy()
    np.testing.assert_allclose(got[:5], [-0.964, -0.762, 0.0, 0.762, 0.964], atol=1e-3)
    np.testing.assert_allclose(got, np.tanh(x.astype(np.float64)), rtol=1e-5, atol=1e-6)


def test_sdpa_softcap_reference_case(T, fusion):
    """transformer.rs test_sdpa_softcap: scores of 10 * scale capped through tanh stay finite; values
    against the closed form."""
    q = np.array([[[[10.0, 0.0], [0.0, 10.0]]]], np.float32)
    v = np.array([[[[1.0, 0.0], [0.0, 1.0]]]], np.float32)
    t = T.Tensor.from_numpy(q).scaled_dot_product_attention(T.Tensor.from_numpy(q), T.Tensor.from_numpy(v), softcap=1.0)
    got = t.to_numpy()
    assert got.shape == (1, 1, 2, 2) and np.all(np.isfinite(got))
    np.testing.assert_allclose(got, _np_sdpa(q, q, v, 1 / np.sqrt(2), softcap=1.0), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("kind", ["bool", "bool_broadcast", "additive", "additive_causal_softcap"])
def test_sdpa_attn_mask(T, fusion, kind):
    """Attention masks (transformer.rs:112-125): Bool (true = attend) and additive, full and
    broadcast over batch and heads, alone and together with the causal mask and a softcap;
    against the float64 closed form.  Every query keeps at least one visible key."""
    rng = np.random.default_rng(61)
    B, H, Sq, Sk, D = 2, 3, 20, 28, 16
    q, k, v = (rng.standard_normal(sh).astype(np.float32) for sh in ((B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D)))
    scale = 1 / np.sqrt(D)
    causal, softcap = False, None
    if kind == "bool":
        mask = rng.random((B, H, Sq, Sk)) < 0.6
        mask[..., 0] = True
    elif kind == "bool_broadcast":
        mask = rng.random((1, 1, Sq, Sk)) < 0.5
        mask[..., 0] = True
    elif kind == "additive":
        mask = rng.standard_normal((B, 1, Sq, Sk)).astype(np.float32)
    else:
        mask = rng.standard_normal((Sq, Sk)).astype(np.float32)
        causal, softcap = True, 5.0
    t = T.Tensor.from_numpy(q).scaled_dot_product_attention(T.Tensor.from_numpy(k), T.Tensor.from_numpy(v), is_causal=causal,
                                                            attn_mask=T.Tensor.from_numpy(mask), softcap=softcap)
    got = t.to_numpy()
    want = _np_sdpa(q, k, v, scale, causal=causal, mask=mask, softcap=softcap)
    assert np.all(np.isfinite(got))
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-5)
    assert not any(n.startswith("flash_fwd") for n in t.kernels())


def test_sdpa_bf16_with_mask_and_softcap_is_the_fused_kernel(T, oracle):
    """tensor/src/transformer.rs:112-132 inside the fused kernel: a Bool mask, an additive bf16
    mask (as a broadcast [B, 1, 1, Sk] view and as a slice of a larger tensor) and a softcap each
    run as ONE flash_fwd kernel, <= 2e-2 against the oracle; the same graphs with the hand-written
    kernels switched off (the composed graph, bf16 scores) agree with it loosely."""
    from morok_amd import synth, uop

    rng = np.random.default_rng(62)
    B, H, S, D = 2, 2, 192, 128
    q, k, v = (synth.to_bf16(rng.standard_normal((B, H, S, D)).astype(np.float32)) for _ in range(3))
    tq, tk, tv = (T.Tensor.from_numpy(a, uop.BF16) for a in (q, k, v))
    scale = 1 / np.sqrt(D)
    mask = rng.random((S, S)) < 0.7
    mask[:, 0] = True
    t = tq.scaled_dot_product_attention(tk, tv, attn_mask=T.Tensor.from_numpy(mask))
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16_ext_bool"), t.kernels()
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, scale, mask=mask))
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # causal + key padding mask [B, 1, 1, S] + softcap, the mask an expand of a [B, S] tensor
    pad = np.ones((B, S), bool)
    pad[0, 150:] = False
    pad[1, 3:40] = False
    tm = T.Tensor.from_numpy(pad).try_reshape([B, 1, 1, S])
    t = tq.scaled_dot_product_attention(tk, tv, is_causal=True, attn_mask=tm, softcap=20.0)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16_ext_bool_cap"), t.kernels()
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, scale, causal=True, mask=pad.reshape(B, 1, 1, S), softcap=20.0))
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # additive bf16 mask that is a slice of a larger tensor in memory: read in place
    big = synth.to_bf16((rng.standard_normal((H, S + 8, S + 64)) * 2).astype(np.float32))
    tm = T.Tensor.from_numpy(big, uop.BF16).try_shrink([(0, H), (8, S + 8), (64, S + 64)])
    t = tq.scaled_dot_product_attention(tk, tv, attn_mask=tm)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16_ext_add"), t.kernels()
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, scale, mask=np.ascontiguousarray(big[:, 8:, 64:])))
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # softcap alone
    t = tq.scaled_dot_product_attention(tk, tv, softcap=1.5)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16_ext_cap"), t.kernels()
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, scale, softcap=1.5))
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    # an f32 mask changes the dtype of the scores: composed graph, as before; so does a key count
    # that is not a multiple of four
    T.set_fusion(False)
    try:
        t = tq.scaled_dot_product_attention(tk, tv, attn_mask=T.Tensor.from_numpy(mask), softcap=1.5)
        loose = synth.from_bf16(t.to_numpy())
        assert not any(n.startswith("flash_fwd") for n in t.kernels())
    finally:
        T.set_fusion(True)
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, scale, mask=mask, softcap=1.5))
    assert np.abs(loose - ref).max() <= 6e-2 * np.abs(ref).max()
    k3, v3 = k[:, :, :190], v[:, :, :190]
    t = tq.scaled_dot_product_attention(T.Tensor.from_numpy(k3, uop.BF16), T.Tensor.from_numpy(v3, uop.BF16),
                                        attn_mask=T.Tensor.from_numpy(mask[:, :190]))
    got = synth.from_bf16(t.to_numpy())
    assert not any(n.startswith("flash_fwd") for n in t.kernels())
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k3, v3, scale, mask=np.ascontiguousarray(mask[:, :190])))
    assert np.abs(got - ref).max() <= 6e-2 * np.abs(ref).max()


def test_sdpa_padded_head_dim_with_mask_and_softcap(T, oracle):
    """A head dim without an instantiation (96) is zero-padded to 128 by the graph builder; mask and
    softcap ride along into the fused kernel."""
    from morok_amd import synth, uop

    rng = np.random.default_rng(63)
    B, H, S, D = 1, 2, 128, 96
    q, k, v = (synth.to_bf16(rng.standard_normal((B, H, S, D)).astype(np.float32)) for _ in range(3))
    mask = rng.random((B, H, S, S)) < 0.5
    mask[..., 0] = True
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16), T.Tensor.from_numpy(v, uop.BF16),
                                                                      attn_mask=T.Tensor.from_numpy(mask), softcap=5.0)
    got = synth.from_bf16(t.to_numpy())
    assert sum(n.startswith("flash_fwd_bf16_ext") for n in t.kernels()) == 1
    ref = synth.from_bf16(oracle.sdpa_bf16_ex(q, k, v, 1 / np.sqrt(D), mask=mask, softcap=5.0))
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()


def test_sdpa_bf16_uses_flash(T, oracle):
    from morok_amd import synth, uop

    rng = np.random.default_rng(29)
    B, H, S, D = 1, 2, 256, 128
    q, k, v = (synth.to_bf16(rng.standard_normal((B, H, S, D)).astype(np.float32)) for _ in range(3))
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(T.Tensor.from_numpy(k, uop.BF16),
                                                                      T.Tensor.from_numpy(v, uop.BF16), is_causal=True)
    got = synth.from_bf16(t.to_numpy())
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd")
    ref = synth.from_bf16(oracle.sdpa_bf16(q, k, v, 1 / np.sqrt(D), True))
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()


def test_matmul_bf16_generated_tensor_core_small_tiles(T, oracle):
    """With the hand-written kernels off, bf16 products whose extents are multiples of 16 (not
    of 128) still take the tensor-core route, on a smaller workgroup tile."""
    from morok_amd import synth, uop

    T.set_fusion(False)
    try:
        for (M, N, K) in ((64, 192, 96), (48, 16, 64), (96, 64, 32)):
            a = synth.normal_bf16((M, K), 51, 0)
            w = synth.normal_bf16((K, N), 51, 1)
            t = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(w, uop.BF16))
            got = synth.from_bf16(t.to_numpy())
            assert t.kernels() == [f"r_tc_{M}_{N}_{K}"]
            ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(w).astype(np.float64)
            assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    finally:
        T.set_fusion(True)


@pytest.mark.parametrize("rows,part,nparts,dtype", [(64, 64, 2, "f32"), (256, 32, 4, "f32"), (48, 8, 2, "f32"), (8, 256, 2, "f32"),
                                                     (64, 64, 2, "bf16"), (30, 64, 2, "f32"), (64, 24, 2, "f32"), (64, 64, 3, "f32"),
                                                     (64, 512, 2, "f32")])
def test_cat_of_computed_parts(T, rows, part, nparts, dtype):
    """cat of parts that are computed (not just loaded) along the innermost axis: the kernel is
    split into one guarded region per part when the parts are equal, a whole number of upcast
    groups and fit the wave renumbering, and falls back to evaluate-and-select otherwise (odd
    row counts, three parts, parts wider than a wave); permuted in front of the store as well.
    All against numpy on the same values."""
    from morok_amd import synth, uop

    rng = np.random.default_rng(rows * 1000 + part * 10 + nparts)
    x = rng.standard_normal((4, rows, part)).astype(np.float32)
    y = rng.standard_normal((4, rows, part)).astype(np.float32)
    if dtype == "bf16":
        xb, yb = synth.to_bf16(x), synth.to_bf16(y)
        x, y = synth.from_bf16(xb), synth.from_bf16(yb)
        tx, ty = T.Tensor.from_numpy(xb, uop.BF16), T.Tensor.from_numpy(yb, uop.BF16)
    else:
        tx, ty = T.Tensor.from_numpy(x), T.Tensor.from_numpy(y)
    exprs = [lambda a, b: a * b - b, lambda a, b: a + b * 2.0, lambda a, b: a * a, lambda a, b: b - a]
    tparts = [(tx.try_mul(ty).try_sub(ty)), (tx.try_add(ty.try_mul(2.0))), (tx.try_mul(tx)), (ty.try_sub(tx))][:nparts]
    want = np.concatenate([f(x, y) for f in exprs[:nparts]], axis=-1)
    t = T.Tensor.cat(tparts, -1)
    got = t.to_numpy()
    assert len(t.kernels()) == 1
    gotf = synth.from_bf16(got) if dtype == "bf16" else got
    tol = 1e-2 if dtype == "bf16" else 1e-6
    np.testing.assert_allclose(gotf, want, rtol=tol, atol=tol)
    tp = T.Tensor.cat(tparts, -1).try_permute([1, 0, 2]).contiguous()
    gp = tp.to_numpy()
    gpf = synth.from_bf16(gp) if dtype == "bf16" else gp
    np.testing.assert_allclose(gpf, want.transpose(1, 0, 2), rtol=tol, atol=tol)


def test_sdpa_bf16_reads_and_writes_views_in_place(T, oracle):
    """q / k / v as column slices of one packed [B*S, 3*H*D] buffer seen as [B, H, S, D], the
    result permuted back to [B*S, H*D]: one attention kernel and no copy kernels, and the bits
    of the attention over dense copies of the same operands."""
    from morok_amd import synth, uop

    B, H, S, D = 2, 3, 192, 128
    hid = H * D
    packed = synth.normal_bf16((B * S, 3 * hid), 41, 0)
    pt = T.Tensor.from_numpy(packed, uop.BF16)

    def head_view(t, i):
        return (t.try_shrink([(0, B * S), (i * hid, (i + 1) * hid)]).try_reshape([B, S, H, D]).try_permute([0, 2, 1, 3]))

    q, k, v = (head_view(pt, i) for i in range(3))
    out = q.scaled_dot_product_attention(k, v, is_causal=True).try_permute([0, 2, 1, 3]).try_reshape([B * S, hid])
    got = out.to_numpy()
    assert out.kernels() == [f"flash_fwd_bf16_strided_{B * H}_{S}_{S}"]
    qn, kn, vn = (np.ascontiguousarray(packed[:, i * hid:(i + 1) * hid].reshape(B, S, H, D).transpose(0, 2, 1, 3))
                  for i in range(3))
    dense = T.Tensor.from_numpy(qn, uop.BF16).scaled_dot_product_attention(
        T.Tensor.from_numpy(kn, uop.BF16), T.Tensor.from_numpy(vn, uop.BF16), is_causal=True)
    want = dense.to_numpy()
    assert dense.kernels()[0].startswith("flash_fwd_bf16_") and "strided" not in dense.kernels()[0]
    assert np.array_equal(got.reshape(B, S, H, D).transpose(0, 2, 1, 3), want)
    ref = synth.from_bf16(oracle.sdpa_bf16(qn, kn, vn, 1 / np.sqrt(D), True))
    assert np.abs(synth.from_bf16(want) - ref).max() <= 2e-2 * np.abs(ref).max()


def test_sdpa_bf16_shared_keys_by_expand(T):
    """Keys and values of one head expanded over all heads: read through zero strides."""
    from morok_amd import synth, uop

    B, H, S, D = 1, 4, 160, 128
    q = synth.normal_bf16((B, H, S, D), 42, 0)
    k1, v1 = synth.normal_bf16((B, 1, S, D), 42, 1), synth.normal_bf16((B, 1, S, D), 42, 2)
    kt = T.Tensor.from_numpy(k1, uop.BF16).try_expand([B, H, S, D])
    vt = T.Tensor.from_numpy(v1, uop.BF16).try_expand([B, H, S, D])
    t = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(kt, vt, is_causal=False)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("flash_fwd_bf16_strided")
    kb, vb = (np.ascontiguousarray(np.broadcast_to(x, (B, H, S, D))) for x in (k1, v1))
    want = T.Tensor.from_numpy(q, uop.BF16).scaled_dot_product_attention(
        T.Tensor.from_numpy(kb, uop.BF16), T.Tensor.from_numpy(vb, uop.BF16), is_causal=False).to_numpy()
    assert np.array_equal(got, want)


def test_sdpa_bf16_views_the_kernel_cannot_take_are_copied(T):
    """A view with an unaligned offset, a transposed head dimension, an attention result with
    two readers, and a view of an unrealised elementwise expression: each falls back to dense
    copies (or the dense layout) and gives the same values."""
    from morok_amd import synth, uop

    B, H, S, D = 1, 2, 128, 128
    big = synth.normal_bf16((B, H, S + 1, D + 4), 43, 0)
    bt = T.Tensor.from_numpy(big, uop.BF16)
    q = synth.normal_bf16((B, H, S, D), 43, 1)
    qt = T.Tensor.from_numpy(q, uop.BF16)
    kv = bt.try_shrink([(0, B), (0, H), (1, S + 1), (4, D + 4)])                 # offset 4 mod 8, row stride 132
    t = qt.scaled_dot_product_attention(kv, kv, is_causal=True)
    got = t.to_numpy()
    assert sum(k.startswith("flash_fwd_bf16_") for k in t.kernels()) == 1 and not any("strided" in k for k in t.kernels())
    kn = np.ascontiguousarray(big[:, :, 1:, 4:])
    want = qt.scaled_dot_product_attention(T.Tensor.from_numpy(kn, uop.BF16), T.Tensor.from_numpy(kn, uop.BF16),
                                           is_causal=True).to_numpy()
    assert np.array_equal(got, want)
    # head dimension not innermost
    kT = T.Tensor.from_numpy(np.ascontiguousarray(kn.transpose(0, 1, 3, 2)), uop.BF16).try_permute([0, 1, 3, 2])
    t2 = qt.scaled_dot_product_attention(kT, kT, is_causal=True)
    assert np.array_equal(t2.to_numpy(), want) and not any("strided" in k for k in t2.kernels())
    # two readers of the attention result: it is kept in its own layout
    a = qt.scaled_dot_product_attention(T.Tensor.from_numpy(kn, uop.BF16), T.Tensor.from_numpy(kn, uop.BF16), is_causal=True)
    both = a.try_permute([0, 2, 1, 3]).try_reshape([B * S, H * D]).try_add(a.try_reshape([B * S, H * D]))
    gb = synth.from_bf16(both.to_numpy())
    assert not any("strided" in k for k in both.kernels())
    wf = synth.from_bf16(want)
    exp = wf.transpose(0, 2, 1, 3).reshape(B * S, H * D) + wf.reshape(B * S, H * D)
    assert np.abs(gb - exp).max() <= 1e-2 * np.abs(exp).max()
    # a slice of an elementwise expression is computed over the slice, not over its base
    e = bt.try_mul(1.0).try_shrink([(0, B), (0, H), (0, S), (0, D)])
    t3 = qt.scaled_dot_product_attention(e, e, is_causal=True)
    kn3 = np.ascontiguousarray(big[:, :, :S, :D])
    want3 = qt.scaled_dot_product_attention(T.Tensor.from_numpy(kn3, uop.BF16), T.Tensor.from_numpy(kn3, uop.BF16),
                                            is_causal=True).to_numpy()
    assert np.array_equal(t3.to_numpy(), want3) and not any("strided" in k for k in t3.kernels())


def test_silu_and_sigmoid(T, oracle):
    rng = np.random.default_rng(31)
    x = (rng.standard_normal(5000) * 4).astype(np.float32)
    got = T.Tensor.from_numpy(x).silu().to_numpy()
    np.testing.assert_allclose(got, oracle.silu_f32(x), rtol=1e-5, atol=1e-6)
    s = T.Tensor.from_numpy(x).sigmoid().to_numpy()
    np.testing.assert_allclose(s, 1 / (1 + np.exp(-x.astype(np.float64))), rtol=1e-5, atol=1e-7)


# ---------------------------------------------------------------- realize / caching
def test_realize_reuses_cached_kernels(T):
    from morok_amd import tensor

    x = np.arange(1000, dtype=np.float32)
    a = T.Tensor.from_numpy(x).try_mul(3.0).try_add(1.0)
    a.realize()
    first = tensor.last_cached_count()
    b = T.Tensor.from_numpy(x + 1).try_mul(3.0).try_add(1.0)
    b.realize()
    assert tensor.last_cached_count() == 1 and first in (0, 1)  # same AST -> same kernel (kernel_cache.rs:87-118)
    np.testing.assert_array_equal(b.to_numpy(), (x + 1) * 3 + 1)
    # realizing again is a no-op; a consumer of a realized tensor reads its buffer
    b.realize()
    assert tensor.last_kernels() == []
    c = b.try_sub(1.0)
    np.testing.assert_array_equal(c.to_numpy(), (x + 1) * 3)
    assert len(c.kernels()) == 1


def test_contiguous_is_a_kernel_boundary(T):
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    t = T.Tensor.from_numpy(x).try_transpose(0, 1).contiguous()
    y = t.try_add(1.0)
    np.testing.assert_array_equal(y.to_numpy(), x.T + 1)
    assert len(y.kernels()) == 2


def test_large_elementwise_bandwidth_shape(T):
    # 64 Mi elements: exercises the 2^31 byte range with int32 element indices
    n = 1 << 26
    from morok_amd import uop

    t = T.Tensor.full([n], 1.5, uop.F32).try_mul(T.Tensor.full([n], 2.0, uop.F32)).contiguous()
    s = t.sum(0)
    assert float(s.to_numpy()) == 3.0 * n


# ---------------------------------------------------------------- realize_binary.rs
_NP_BIN = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "fdiv": np.divide}


@pytest.mark.parametrize("case", GOLD["realize_binary"]["cases"], ids=lambda c: c["name"])
def test_realize_binary_cases(T, case):
    a, b = f32(case["a"]), f32(case["b"])
    got = T.Tensor.from_numpy(a).binary(case["op"], T.Tensor.from_numpy(b)).to_numpy()
    want = f32(case["expected"]) if "expected" in case else _NP_BIN[case["op"]](a, b)
    np.testing.assert_allclose(got, want, atol=case["tol"], rtol=0)


@pytest.mark.parametrize("case", GOLD["realize_binary"]["chained"], ids=lambda c: c["name"])
def test_realize_chained_expressions(T, case):
    t = {k: T.Tensor.from_numpy(f32(case[k])) for k in "abcde" if k in case}
    expr = {"add_mul": lambda: (t["a"] + t["b"]) * t["c"], "mul_add": lambda: t["a"] * t["b"] + t["c"],
            "sub_div": lambda: (t["a"] - t["b"]) / t["c"],
            "complex": lambda: ((t["a"] + t["b"]) * t["c"] - t["d"]).try_div(t["e"])}[case["name"]]()
    got = expr.to_numpy()
    assert len(expr.kernels()) == 1          # one fused elementwise kernel
    np.testing.assert_allclose(got, f32(case["expected"]), atol=case["tol"], rtol=0)


def test_embedding_out_of_range_index_reads_zero(T):
    """An index outside the vocabulary selects nothing (the reference gathers by comparing
    against arange(vocab)); on the GPU it must in particular not read out of bounds."""
    w = np.arange(12, dtype=np.float32).reshape(3, 4) + 1
    idx = np.array([2, -1, 0, 3, 7_000_000], dtype=np.int32)
    got = T.Tensor.from_numpy(w).embedding(T.Tensor.from_numpy(idx)).to_numpy()
    want = np.stack([w[2], np.zeros(4), w[0], np.zeros(4), np.zeros(4)]).astype(np.float32)
    np.testing.assert_array_equal(got, want)


def test_empty_tensors_and_empty_cat_parts(T):
    e = T.Tensor.from_numpy(np.zeros((0, 4), np.float32))
    assert e.try_add(1.0).to_numpy().shape == (0, 4)
    x = np.arange(8, dtype=np.float32).reshape(2, 4)
    c = T.Tensor.cat([T.Tensor.from_numpy(x), e, T.Tensor.from_numpy(x + 10)], 0)
    np.testing.assert_array_equal(c.to_numpy(), np.concatenate([x, x + 10], 0))


def test_split_reduction_values(T):
    """Long reductions (>= 32768 inputs per output), ragged segment ends included: few outputs share
    each output between the 16 waves of a workgroup in one kernel, a single output of 2^21 inputs
    also splits into segments folded by a second kernel."""
    rng = np.random.default_rng(41)
    x = rng.standard_normal((3, 100003)).astype(np.float32)
    t = T.Tensor.from_numpy(x)
    s = t.sum(1)
    np.testing.assert_allclose(s.to_numpy(), x.astype(np.float64).sum(1), rtol=1e-4, atol=1e-2)
    assert s.kernels() == ["r_3_g100003_l16"]
    np.testing.assert_array_equal(t.max(1).to_numpy(), x.max(1))
    y = rng.standard_normal((1 << 21,)).astype(np.float32)
    ty = T.Tensor.from_numpy(y).sum(0)
    np.testing.assert_allclose(ty.to_numpy(), y.astype(np.float64).sum(), rtol=1e-4, atol=1e-2)
    assert len(ty.kernels()) == 2
    z = rng.standard_normal((2, 200, 300)).astype(np.float32)   # several reduced axes, strided
    np.testing.assert_allclose(T.Tensor.from_numpy(z).sum([1, 2]).to_numpy(), z.astype(np.float64).sum((1, 2)), rtol=1e-4,
                               atol=1e-2)
    np.testing.assert_allclose(T.Tensor.from_numpy(z).try_permute([1, 0, 2]).sum([0, 2]).to_numpy(),
                               z.astype(np.float64).sum((1, 2)), rtol=1e-4, atol=1e-2)


# ---------------------------------------------------------------- generated kernels stay inside their inputs
def _guarded(dev, arr):
    """A tensor over a view that has NaNs right in front of and right behind its data in the
    same allocation."""
    import morok_amd

    from morok_amd import uop

    pad = 4096
    raw = np.full(pad * 2 + arr.nbytes, 0xFF, np.uint8)      # 0xFFFFFFFF = NaN in f32, -1 in int32
    raw[pad:pad + arr.nbytes] = np.frombuffer(np.ascontiguousarray(arr).tobytes(), np.uint8)
    base = morok_amd.Buffer.from_numpy(raw, dev.device_id)
    dt = {np.dtype(np.float32): uop.F32, np.dtype(np.int32): uop.I32}[arr.dtype]
    return base, base.view(pad, arr.nbytes), dt


def test_generated_kernels_do_not_read_past_their_inputs(T, dev):
    """Movement ops become index arithmetic inside the consuming kernel; edges of shrink, cat,
    gather (clamped rows, masked out-of-range indices), reductions and odd widths must not pull
    in what lies next to the data (NaNs here, which would poison sums and selections)."""
    rng = np.random.default_rng(31)
    x = rng.standard_normal((37, 53)).astype(np.float32)
    keep, view, dt = _guarded(dev, x)
    t = T.Tensor.from_buffer(view, x.shape, dt)
    # reduce over both axes, odd extents
    np.testing.assert_allclose(t.sum([1]).to_numpy(), x.sum(1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(t.sum([0]).to_numpy(), x.sum(0), rtol=1e-5, atol=1e-5)
    # shrink to the last rows / columns, transpose, cat of the two edges
    a = t.try_shrink([(30, 37), (40, 53)])
    b = t.try_shrink([(0, 7), (0, 13)])
    got = T.Tensor.cat([a, b], 1).try_transpose(0, 1).contiguous().to_numpy()
    np.testing.assert_array_equal(got, np.concatenate([x[30:37, 40:53], x[0:7, 0:13]], 1).T)
    # wide rows (vector loads) with a tail
    y = rng.standard_normal((9, 1027)).astype(np.float32)
    keep2, view2, _ = _guarded(dev, y)
    ty = T.Tensor.from_buffer(view2, y.shape, dt)
    np.testing.assert_allclose(ty.try_mul(ty).sum([1]).to_numpy(), (y * y).sum(1), rtol=1e-5)
    np.testing.assert_allclose(ty.softmax(-1).to_numpy(), np.exp(y - y.max(1, keepdims=True)) /
                               np.exp(y - y.max(1, keepdims=True)).sum(1, keepdims=True), rtol=1e-5, atol=1e-9)
    # gather: first row, last row and out-of-range indices (which select nothing)
    w = rng.standard_normal((11, 24)).astype(np.float32)
    keep3, view3, _ = _guarded(dev, w)
    tw = T.Tensor.from_buffer(view3, w.shape, dt)
    idx = np.array([0, 10, 11, -1, 5, 1000], np.int32)
    want = np.where(((idx >= 0) & (idx < 11))[:, None], w[np.clip(idx, 0, 10)], 0.0)
    np.testing.assert_array_equal(tw.embedding(T.Tensor.from_numpy(idx)).to_numpy(), want)
    del keep, keep2, keep3


@pytest.mark.parametrize("npdt,tag", [(np.uint8, "U8"), (np.int8, "I8"), (np.int16, "I16"), (np.uint16, "U16")])
def test_narrow_integer_arithmetic_wraps(T, npdt, tag):
    """8- and 16-bit integer elementwise kernels (vectorised 16 / 8 wide): results wrap modulo
    2^bits like the reference's C backend, bit-exact against numpy."""
    from morok_amd import uop

    dt = getattr(uop, tag)
    rng = np.random.default_rng(41)
    info = np.iinfo(npdt)
    a = rng.integers(info.min, info.max, size=(33, 64), endpoint=True).astype(npdt)
    b = rng.integers(info.min, info.max, size=(33, 64), endpoint=True).astype(npdt)
    ta, tb = T.Tensor.from_numpy(a, dt), T.Tensor.from_numpy(b, dt)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(ta.try_add(tb).to_numpy(), (a + b).astype(npdt))
        np.testing.assert_array_equal(ta.try_mul(tb).try_sub(ta).to_numpy(), (a * b - a).astype(npdt))
    np.testing.assert_array_equal(ta.maximum(tb).to_numpy(), np.maximum(a, b))


def test_more_than_2_pow_31_elements(T, dev):
    """Index arithmetic switches to 64 bits when a kernel's iteration space or one of its
    inputs has 2^31 elements or more: a broadcast view of 2^32 elements reduced by rows, and a
    real 2^31 + 64 byte tensor through an elementwise kernel (first, last and middle checked)."""
    from morok_amd import uop

    T.set_fusion(False)
    s = T.Tensor.full([1 << 16, 1 << 16], 0.5, uop.F32).sum([1])
    got = s.to_numpy()
    assert got.shape == (1 << 16,) and np.all(got == 32768.0)

    n = (1 << 31) + 64
    x = np.empty(n, np.uint8)
    x[:] = np.arange(n, dtype=np.uint64).astype(np.uint8)       # value = index mod 256
    t = T.Tensor.from_numpy(x, uop.U8)
    y = t.try_add(T.Tensor.const(3, uop.U8)).to_numpy()
    assert y.shape == (n,)
    for lo in (0, (1 << 31) - 128, n - 256, 1_234_567_890):
        np.testing.assert_array_equal(y[lo:lo + 128], ((np.arange(lo, lo + 128) + 3) % 256).astype(np.uint8))
    T.set_fusion(True)


_NP = {"BOOL": np.bool_, "I8": np.int8, "U8": np.uint8, "I16": np.int16, "U16": np.uint16, "I32": np.int32,
       "U32": np.uint32, "I64": np.int64, "U64": np.uint64, "F16": np.float16, "F32": np.float32, "F64": np.float64}


def _values(name, shape, rng):
    """In-range test values for a dtype (small magnitudes so every cast below is defined)."""
    if name == "BOOL":
        return rng.integers(0, 2, size=shape).astype(np.bool_)
    if name.startswith("U"):
        return rng.integers(0, 100, size=shape).astype(_NP[name])
    if name.startswith("I"):
        return rng.integers(-100, 100, size=shape).astype(_NP[name])
    return (rng.integers(-400, 400, size=shape) / 4.0).astype(_NP[name])   # quarter steps: exact in f16


@pytest.mark.parametrize("src", list(_NP))
def test_cast_matrix(T, src):
    """Every dtype to every other through a generated kernel, against numpy's C-style
    conversions (float -> integer truncates toward zero, anything -> bool is != 0, a negative
    integer -> unsigned wraps); values are chosen in range of every target."""
    from morok_amd import uop

    rng = np.random.default_rng(51)
    x = _values(src, (5, 48), rng)
    t = T.Tensor.from_numpy(x, getattr(uop, src))
    for dst, npdst in _NP.items():
        xs, ts = x, t
        if src[0] == "F" and dst[0] == "U":
            # a negative floating value has no defined conversion to an unsigned type in C
            xs = np.abs(x)
            ts = T.Tensor.from_numpy(xs, getattr(uop, src))
        got = ts.cast(getattr(uop, dst)).to_numpy()
        if dst == "BOOL":
            want = xs != 0
        elif dst[0] == "U" and src[0] == "I":
            want = xs.astype(np.int64).astype(npdst)     # negative -> unsigned wraps modulo 2^bits
        else:
            want = xs.astype(npdst)
        np.testing.assert_array_equal(got, want, err_msg=f"{src} -> {dst}")


@pytest.mark.parametrize("name", ["I8", "U8", "I16", "U16", "I32", "U32", "I64", "U64", "F16", "F64"])
def test_reductions_and_comparisons_across_dtypes(T, name):
    from morok_amd import uop

    rng = np.random.default_rng(52)
    a, b = _values(name, (7, 300), rng), _values(name, (7, 300), rng)
    ta, tb = T.Tensor.from_numpy(a, getattr(uop, name)), T.Tensor.from_numpy(b, getattr(uop, name))
    np.testing.assert_array_equal(ta.max([1]).to_numpy(), a.max(1))
    np.testing.assert_array_equal(ta.where(ta.binary("lt", tb), tb).to_numpy(), np.where(a < b, a, b))
    s = ta.sum([1]).to_numpy()
    if name[0] in "IU":
        assert np.array_equal(s.astype(np.int64), a.astype(np.int64).sum(1))   # sums promote, no wrap at these sizes
    else:
        np.testing.assert_allclose(s.astype(np.float64), a.astype(np.float64).sum(1), rtol=2e-3 if name == "F16" else 1e-12)


def _random_graph(T, rng, x_np, x_t):
    """A random chain of movement and elementwise ops applied to (numpy array, tensor) alike."""
    a, t = x_np, x_t
    for _ in range(int(rng.integers(2, 6))):
        kind = rng.choice(["permute", "reshape", "shrink", "expand", "cat", "add", "mul", "flipcat", "contig"])
        if kind == "permute" and a.ndim >= 2:
            perm = list(rng.permutation(a.ndim))
            a, t = np.transpose(a, perm), t.try_permute([int(p) for p in perm])
        elif kind == "reshape":
            n = a.size
            divs = [d for d in (1, 2, 3, 4, 6, 8, 12, 16, 24) if n % d == 0]
            d0 = int(rng.choice(divs))
            rest = n // d0
            divs2 = [d for d in (1, 2, 3, 4, 8) if rest % d == 0]
            d1 = int(rng.choice(divs2))
            shape = [d0, d1, rest // d1]
            a, t = np.ascontiguousarray(a).reshape(shape), t.try_reshape(shape)
        elif kind == "shrink" and a.size > 1:
            rngs = []
            for s in a.shape:
                lo = int(rng.integers(0, max(1, s // 2)))
                hi = int(rng.integers(lo + 1, s + 1))
                rngs.append((lo, hi))
            a, t = a[tuple(slice(lo, hi) for lo, hi in rngs)], t.try_shrink(rngs)
        elif kind == "expand" and a.size <= 4096:
            a, t = np.broadcast_to(a[None], (3,) + a.shape), t.try_reshape([1] + list(a.shape)).try_expand([3] + list(a.shape))
        elif kind == "cat" and a.size <= 8192:
            ax = int(rng.integers(0, a.ndim))
            a, t = np.concatenate([a, a * 2], ax), T.Tensor.cat([t, t.try_add(t)], ax)
        elif kind == "flipcat" and a.ndim >= 1 and a.shape[-1] >= 2:
            h = a.shape[-1] // 2
            lo = [(0, s) for s in a.shape[:-1]]
            a2 = np.concatenate([a[..., h:], a[..., :h]], -1)
            t = T.Tensor.cat([t.try_shrink(lo + [(h, a.shape[-1])]), t.try_shrink(lo + [(0, h)])], a.ndim - 1)
            a = a2
        elif kind == "add":
            a, t = a + 1.5, t.try_add(T.Tensor.const(1.5))
        elif kind == "mul":
            a, t = a * a, t.try_mul(t)
        elif kind == "contig":
            a, t = np.ascontiguousarray(a), t.contiguous()
    return a, t


@pytest.mark.parametrize("seed", range(60))
def test_random_movement_chains(T, seed):
    """Random chains of reshape / permute / shrink / expand / cat with arithmetic in between,
    realised as generated kernels (vector loads where the layout allows, scalar otherwise),
    against numpy on the same chain; then reduced over a random axis."""
    rng = np.random.default_rng(1000 + seed)
    shape = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 24])) for _ in range(int(rng.integers(1, 5)))]
    x = rng.integers(-8, 8, size=shape).astype(np.float32)        # small integers: every result is exact
    a, t = _random_graph(T, rng, x, T.Tensor.from_numpy(x))
    assert t.shape == a.shape
    np.testing.assert_array_equal(t.to_numpy(), a)
    if a.ndim:
        ax = int(rng.integers(0, a.ndim))
        np.testing.assert_array_equal(t.sum([ax]).to_numpy(), a.sum(ax))


@pytest.mark.parametrize("seed", range(24))
def test_random_movement_chains_power_of_two_shapes(T, seed):
    """The same with extents that are powers of two up to 128: whole upcast groups, whole waves,
    the shapes on which the generator takes its vector-load, split-group and per-part paths."""
    rng = np.random.default_rng(50000 + seed)
    shape = [int(rng.choice([1, 2, 4, 8, 16, 32, 64, 128])) for _ in range(int(rng.integers(1, 5)))]
    while np.prod(shape) > 1 << 20:
        shape[int(rng.integers(0, len(shape)))] = 2
    x = rng.integers(-8, 8, size=shape).astype(np.float32)
    a, t = _random_graph(T, rng, x, T.Tensor.from_numpy(x))
    assert t.shape == a.shape
    np.testing.assert_array_equal(t.to_numpy(), a)
    if a.ndim:
        ax = int(rng.integers(0, a.ndim))
        np.testing.assert_array_equal(t.sum([ax]).to_numpy(), a.sum(ax))


def test_linear_reads_the_weight_as_stored(T, oracle):
    """x.linear(w) with w [out, in] (tensor/src/nn/linear.rs:39-41): one product kernel that reads
    the weight in place, the bits of the product with the transposed copy, and within the GEMM
    tolerance of the oracle; also under the residual add and with a ragged K."""
    from morok_amd import synth, uop

    T.set_fusion(True)
    for (M, K, N) in ((512, 256, 768), (300, 200, 264)):
        x, w, h = synth.normal_bf16((M, K), 9, 11), synth.normal_bf16((N, K), 9, 12), synth.normal_bf16((M, N), 9, 13)
        tx, tw, th = (T.Tensor.from_numpy(t, uop.BF16) for t in (x, w, h))
        y = tx.linear(tw)
        got = y.to_numpy()
        assert y.kernels() == [f"gemm_bf16_nt_{M}_{N}_{K}"]
        wt = np.ascontiguousarray(w.T)
        want = tx.matmul(T.Tensor.from_numpy(wt, uop.BF16)).to_numpy()
        assert np.array_equal(got, want)
        ref = synth.from_bf16(oracle.gemm_bf16(x, wt))
        assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
        r = th.try_add(tx.linear(tw))
        got_r = r.to_numpy()
        assert r.kernels() == [f"gemm_bf16_nt_residual_{M}_{N}_{K}"]
        assert np.array_equal(got_r, synth.to_bf16(synth.from_bf16(got) + synth.from_bf16(h)))


def test_linear_with_bias_is_one_kernel(T, oracle):
    """x.linear(w, bias) in bf16 with the parameters in memory (tensor/src/nn/linear.rs:39-41): one product kernel
    that adds the bias in its epilogue, for a prefill-sized and a decode-sized x; the bits of the unfused graph."""
    from morok_amd import synth, uop

    for (M, K, N) in ((300, 200, 264), (8, 1024, 520), (1, 512, 4100)):
        x, w, b = synth.normal_bf16((M, K), 9, 21), synth.normal_bf16((N, K), 9, 22), synth.normal_bf16((N,), 9, 23)
        T.set_fusion(True)
        y = T.Tensor.from_numpy(x, uop.BF16).linear(T.Tensor.from_numpy(w, uop.BF16), T.Tensor.from_numpy(b, uop.BF16))
        got = y.to_numpy()
        assert y.kernels() == [f"gemm_bf16_nt_bias_{M}_{N}_{K}"]
        ref = synth.from_bf16(oracle.gemm_bf16(x, np.ascontiguousarray(w.T))) + synth.from_bf16(b)[None, :]
        assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
        p = T.Tensor.from_numpy(x, uop.BF16).linear(T.Tensor.from_numpy(w, uop.BF16)).to_numpy()
        assert np.array_equal(got, synth.to_bf16(synth.from_bf16(p) + synth.from_bf16(b)[None, :]))


def test_matmul_bf16_residual_add_is_fused(T):
    """x + a @ w in bf16 with no other reader of the product: one kernel (the product kernel
    with the residual epilogue), on either side of the add and through contiguous(); the same
    bits as with the hand-written kernels' fusion of the add left out; a product with two
    readers is kept and added separately."""
    from morok_amd import synth, uop

    M, K, N = 256, 192, 384
    a, w, x = synth.normal_bf16((M, K), 9, 1), synth.normal_bf16((K, N), 9, 2), synth.normal_bf16((M, N), 9, 3)
    ta, tw, tx = (T.Tensor.from_numpy(t, uop.BF16) for t in (a, w, x))
    T.set_fusion(True)
    left = tx.try_add(ta.matmul(tw)).contiguous()
    got_l = left.to_numpy()
    assert left.kernels() == [f"gemm_bf16_residual_{M}_{N}_{K}"]
    right = ta.matmul(tw).try_add(tx)
    got_r = right.to_numpy()
    assert right.kernels() == [f"gemm_bf16_residual_{M}_{N}_{K}"]
    assert np.array_equal(got_l, got_r)
    prod = ta.matmul(tw)
    separate = synth.to_bf16(synth.from_bf16(prod.to_numpy()) + synth.from_bf16(x))
    assert np.array_equal(got_l, separate)
    mm = ta.matmul(tw)
    both = tx.try_add(mm).try_mul(mm)                      # the product has two readers
    gb = both.to_numpy()
    assert not any(k.startswith("gemm_bf16_residual") for k in both.kernels())
    pf = synth.from_bf16(prod.to_numpy())
    want = synth.from_bf16(synth.to_bf16(pf + synth.from_bf16(x)))
    assert np.abs(synth.from_bf16(gb) - want * pf).max() <= 2e-2 * np.abs(want * pf).max()
    bx = T.Tensor.from_numpy(synth.normal_bf16((1, N), 9, 4), uop.BF16)
    bc = ta.matmul(tw).try_add(bx)                          # a broadcast operand is not a residual
    bc.realize()
    assert not any(k.startswith("gemm_bf16_residual") for k in bc.kernels())


def test_matmul_bf16_few_rows_uses_split_k(T, oracle):
    """A handful of rows against a large weight matrix through the tensor API: the scheduler
    adds the split-K scratch to the plan as an intermediate buffer."""
    from morok_amd import synth, uop

    T.set_fusion(True)
    rng = np.random.default_rng(61)
    a = synth.to_bf16(rng.standard_normal((4, 2048), dtype=np.float32))
    w = synth.to_bf16(rng.standard_normal((2048, 1024), dtype=np.float32))
    c = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(w, uop.BF16))
    got = synth.from_bf16(c.to_numpy())
    ref = synth.from_bf16(oracle.gemm_bf16(a, w))
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    assert c.kernels() == ["gemm_bf16_4_1024_2048_splitk"]


def test_matmul_bf16_generated_tensor_core(T, oracle):
    """With the hand-written kernels off, a bf16 matmul whose N and K are multiples of 8 takes
    the generated tensor-core kernel (WMMA staged through local memory; extents the workgroup
    tile does not divide are padded); other shapes keep the generic reduce kernel.  Same numerics policy as the hand-written GEMM: exact
    products, f32 accumulation, one rounding."""
    from morok_amd import synth, uop

    T.set_fusion(False)
    rng = np.random.default_rng(71)
    for (M, N, K), tc in (((256, 128, 96), True), ((128, 256, 1024), True), ((96, 128, 64), True), ((100, 128, 64), True), ((96, 128, 40), True),
                           ((3, 8, 8), True), ((100, 132, 64), False), ((96, 128, 36), False)):
        a = synth.to_bf16(rng.standard_normal((M, K), dtype=np.float32))
        w = synth.to_bf16(rng.standard_normal((K, N), dtype=np.float32))
        c = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(w, uop.BF16))
        got = synth.from_bf16(c.to_numpy())
        ref = synth.from_bf16(oracle.gemm_bf16(a, w))
        assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
        assert (c.kernels() == [f"r_tc_{M}_{N}_{K}"]) == tc, c.kernels()
        if tc:
            assert "__builtin_amdgcn_mfma" in T.last_kernel_sources()[0] and "__shared__" in T.last_kernel_sources()[0]
    T.set_fusion(True)


# ---------------------------------------------------------------- Tensor::to / COPY plan items
def test_host_tensors_through_device_copies(T, oracle):
    """Host-resident tensors (Tensor::from_slice), moved with to("HIP:0") as lazy COPY nodes that
    the plan executes in order with its kernels (tensor/src/lib.rs:479-486,
    tensor/src/realize.rs:1002-1011), on the reference's own matmul / softmax cases."""
    for key in ("matmul_2x2", "matmul_3x3"):
        g = GOLD[key]
        a, b = T.Tensor.from_slice(f32(g["a"])), T.Tensor.from_slice(f32(g["b"]))
        assert a.device == "CPU"
        c = a.to("HIP:0").matmul(b.to("HIP:0"))
        got = c.to_numpy()
        assert [k.split("_")[0] for k in c.kernels()] == ["copy", "copy", "r"]
        np.testing.assert_allclose(got, f32(g["expected"]), atol=g["tol"])
    # closed-form generators at 256 (matmul.rs:669-677), result copied back to the CPU device
    n = 256
    x = np.arange(n * n, dtype=np.int64)
    a = ((x % 31) * 0.05 - 0.8).astype(np.float32).reshape(n, n)
    b = ((x % 37) * 0.04 - 0.7).astype(np.float32).reshape(n, n)
    c = T.Tensor.from_slice(a).to("HIP:0").matmul(T.Tensor.from_slice(b).to("HIP:0")).to("CPU")
    assert c.device == "CPU"
    got = c.as_vec().reshape(n, n)
    assert c.kernels()[-1].startswith("copy_d2h")
    ref = oracle.matmul_f32(a, b)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())
    # softmax over host data: rows sum to one and match the oracle
    from morok_amd import synth

    s = synth.normal((64, 1000), 2, 0, sigma=2.0)
    p = T.Tensor.from_slice(s).to("HIP:0").softmax(-1).to("CPU").to_numpy()
    ref = oracle.softmax_f32(s)
    np.testing.assert_allclose(p, ref, rtol=1e-5, atol=1e-9)
    assert np.abs(p.sum(-1) - 1).max() < 1e-4


def test_prepared_plan_reuploads_host_data_on_every_execute(T):
    """The copy is an item of the plan, not a side effect of scheduling: executing a prepared plan
    twice uploads twice, so each run starts from the host bytes even if the device copy of the
    input was overwritten in between (here: by the memory planner handing its block on)."""
    x = np.arange(4096, dtype=np.float32)
    t = T.Tensor.from_slice(x).to("HIP:0").try_mul(3.0).try_add(1.0)
    plan = t.prepare()
    names = [plan.kernel_name(i) for i in range(plan.kernel_count)]
    assert names[0] == "copy_h2d_16384" and len(names) == 2
    for _ in range(2):
        plan.execute()
        np.testing.assert_array_equal(t.to_numpy(), x * 3 + 1)
    # bf16 GEMM of host operands lands on the hand-written kernel after two copies
    from morok_amd import synth, uop

    a, b = synth.normal_bf16((256, 128), 7, 0), synth.normal_bf16((128, 256), 7, 1)
    c = T.Tensor.from_slice(a, uop.BF16).to("HIP:0").matmul(T.Tensor.from_slice(b, uop.BF16).to("HIP:0"))
    direct = T.Tensor.from_numpy(a, uop.BF16).matmul(T.Tensor.from_numpy(b, uop.BF16)).to_numpy()
    assert np.array_equal(c.to_numpy(), direct) and c.kernels()[-1].startswith("gemm_bf16")


# ---------------------------------------------------------------- launch dims from get_grouped_dims
@pytest.mark.parametrize("shape", [(300, 1024), (70000, 1024), (66000, 2, 512), (2, 3, 5, 1024), (70001, 256)])
def test_regrouped_launch_dims_index_exactly(T, shape):
    """Grids come from get_grouped_dims (gidx0 = innermost axis, rows on y until they exceed 65535,
    then regrouped into x and recovered with mod / div): index work is bit-exact, so an integer
    kernel whose value encodes its own position must match numpy for every element."""
    n = int(np.prod(shape))
    x = (np.arange(n, dtype=np.int64) * 2654435761 % 2147483647).astype(np.int32).reshape(shape)
    t = T.Tensor.from_numpy(x)
    got = t.binary("xor", T.Tensor.from_numpy(np.full(shape[-1], 0x5A5A5A5A, np.int32))).binary("add", t).to_numpy()
    want = (x ^ np.int32(0x5A5A5A5A)) + x
    assert np.array_equal(got, want)
    # and through a transposed read (the index of every axis matters, not only the flat one)
    if len(shape) == 2 and shape[0] >= 66000:
        small = x[:, :8].copy()
        tt = T.Tensor.from_numpy(np.ascontiguousarray(small.T)).try_transpose(0, 1).try_add(T.Tensor.from_numpy(small))
        assert np.array_equal(tt.to_numpy(), small + small)


# ---------------------------------------------------------------- GROUP reduce through local memory
@pytest.mark.parametrize("shape,axis", [((64, 8192), 1), ((2048, 1024), 1), ((8, 1 << 20), 1), ((3, 5, 4100), 2),
                                        ((1 << 21,), 0), ((17, 9000), 1), ((4, 70001), 1)])
@pytest.mark.parametrize("op", ["sum", "max"])
def test_grouped_reductions_match_float64(T, fusion, oracle, shape, axis, op):
    """Reductions with few outputs share each output between the waves of a workgroup (local memory
    + barrier), split or unsplit: <= 1e-4 relative against float64 for sums (north-star tolerance for
    f32 reductions), exact for maxima; ragged extents exercise the masked tail blocks."""
    from morok_amd import synth

    x = synth.normal(shape, 31, len(shape), sigma=1.0) + np.float32(0.25)
    t = T.Tensor.from_numpy(x)
    got = (t.sum(axis) if op == "sum" else t.max(axis)).to_numpy()
    if op == "sum":
        ref = x.astype(np.float64).sum(axis)
        scale = np.abs(x.astype(np.float64)).sum(axis)   # condition of the sum: |error| <= 1e-4 * sum |x|
        assert np.all(np.abs(got - ref) <= 1e-4 * np.maximum(np.abs(ref), 1e-3 * scale))
    else:
        assert np.array_equal(got, x.max(axis))
    if len(shape) == 2 and op == "sum" and shape[1] <= 8192:
        # the oracle's softmax holds the same row sums: sum(exp(x - max)) is its normaliser
        p = oracle.softmax_f32(x)
        e = np.exp(x - x.max(1, keepdims=True))
        np.testing.assert_allclose((T.Tensor.from_numpy(e).sum(1).to_numpy())[:, None] * p, e, rtol=2e-5, atol=1e-9)


# ---------------------------------------------------------------- reductions that keep the contiguous axis
@pytest.mark.parametrize("shape,axis,kernels", [((8192, 4096), 0, 2), ((4, 2048, 256), 1, 2), ((300, 1000), 0, 2), ((129, 64), 0, 1),
                                                ((6, 500, 33, 16), 1, 2), ((2, 4096, 8, 64), (1, 2), 2), ((100, 4096), 0, 1)])
@pytest.mark.parametrize("op", ["sum", "max"])
def test_column_reductions(T, shape, axis, kernels, op):
    """A fold that keeps the innermost axis (column sums, a fold over a middle axis) runs with the
    lanes along the kept axis, and splits the outermost reduce axis over more work-items when the
    outputs alone would not fill the chip (two kernels, partials as [segment][output])."""
    from morok_amd import synth

    x = synth.normal(shape, 33, len(shape)) + np.float32(0.25)
    t = T.Tensor.from_numpy(x)
    got = (t.sum(axis) if op == "sum" else t.max(axis)).to_numpy()
    names = T.last_kernels()
    assert len(names) == kernels                                     # an odd or short reduce axis is not split
    assert not any("_g" in nm for nm in names)                       # no wave-per-output kernel
    if op == "sum":
        ref = x.astype(np.float64).sum(axis)
        scale = np.abs(x.astype(np.float64)).sum(axis)
        assert np.all(np.abs(got - ref) <= 1e-4 * np.maximum(np.abs(ref), 1e-3 * scale))
    else:
        assert np.array_equal(got, x.max(axis))


def test_column_reduction_integers_and_bf16(T):
    from morok_amd import synth, uop

    xi = synth.randint((1024, 512), 34, 0, 1000).astype(np.int32) - 500
    assert np.array_equal(T.Tensor.from_numpy(xi).sum(0).to_numpy(), xi.sum(0, dtype=np.int32))
    assert len(T.last_kernels()) == 2
    xb = synth.normal_bf16((512, 2048), 34, 1)
    got = synth.from_bf16(T.Tensor.from_numpy(xb, uop.BF16).sum(0).to_numpy())
    ref = synth.from_bf16(xb).astype(np.float64).sum(0)
    assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(np.abs(ref), 1.0))   # one bf16 rounding of an f32 sum


# ---------------------------------------------------------------- row-resident reduce + elementwise
@pytest.mark.parametrize("rows,cols", [(256, 4096), (1000, 512), (128, 8192), (300, 1024), (130, 64 * 4)])
def test_row_resident_norm_kernels(T, oracle, rows, cols, monkeypatch):
    """rms_norm (and anything of its shape: an elementwise kernel fed by a keepdim reduction over the
    last axis of its own input) runs as ONE kernel that folds a row and produces it from the same
    loads.  Against the oracle's rms_norm, and against the two-kernel path, from which it differs only
    in the order of the row sum."""
    from morok_amd import synth, uop

    x = synth.normal((rows, cols), 81, 0, sigma=1.5)
    t = T.Tensor.from_numpy(x).rms_norm(-1, 1e-5)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("rE_"), t.kernels()
    ref = oracle.rms_norm_f32(x, 1e-5)
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)
    monkeypatch.setenv("MOROK_NO_ROW_FUSION", "1")
    t2 = T.Tensor.from_numpy(x).rms_norm(-1, 1e-5)
    two = t2.to_numpy()
    assert len(t2.kernels()) == 2
    np.testing.assert_allclose(got, two, rtol=2e-6, atol=1e-7)
    monkeypatch.delenv("MOROK_NO_ROW_FUSION")
    # bf16 with a weight, as the decoder block uses it, against the oracle's bf16 stage
    xb, wb = synth.normal_bf16((rows, cols), 82, 0), synth.to_bf16(1.0 + synth.normal((cols,), 82, 1, sigma=0.1))
    tb = T.Tensor.from_numpy(xb, uop.BF16).rms_norm(-1, 1e-6).try_mul(T.Tensor.from_numpy(wb, uop.BF16)).cast(uop.BF16)
    gb = tb.to_numpy()
    assert len(tb.kernels()) == (1 if (cols // 8) % 64 == 0 else 2)   # whole waves of 16-byte vectors per row, or two kernels
    rb = oracle.rms_norm_weight_bf16(xb, wb, 1e-6)
    d = np.abs(gb.astype(np.int32) - rb.astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= 0.01 * d.size      # a bf16 ulp where the f32 sums round apart
    # a row maximum consumed by its own row: x - max(x)
    m = T.Tensor.from_numpy(x)
    sm = m.try_sub(m.max(1, keepdim=True))
    assert np.array_equal(sm.to_numpy(), x - x.max(1, keepdims=True)) and len(sm.kernels()) == 1


@pytest.mark.parametrize("rows,cols,vocab", [(256, 4096, 1000), (130, 512, 37), (1024, 1024, 5)])
def test_row_resident_kernel_writes_the_rows_it_looked_up(T, rows, cols, vocab, monkeypatch):
    """An embedding lookup the caller wants in memory (`contiguous()`) in front of a row-resident
    normalisation: the normalisation's kernel looks the rows up itself and writes them as a second
    output.  Both results carry the bits of the two-kernel path, the looked-up tensor is usable
    afterwards (read back, and as an operand of a later kernel)."""
    from morok_amd import synth, uop

    emb = synth.normal_bf16((vocab, cols), 83, 0)
    tok = synth.randint((rows,), 83, 1, vocab)
    wb = synth.to_bf16(1.0 + synth.normal((cols,), 83, 2, sigma=0.1))

    def run():
        h = T.Tensor.from_numpy(emb, uop.BF16).embedding(T.Tensor.from_numpy(tok)).contiguous()
        xn = h.rms_norm(-1, 1e-6).try_mul(T.Tensor.from_numpy(wb, uop.BF16)).cast(uop.BF16)
        a = xn.to_numpy()
        names = list(xn.kernels())
        later = h.try_add(xn).to_numpy()          # h is read from memory here
        return a, h.to_numpy(), later, names, list(T.last_kernels())

    a, h, later, names, later_names = run()
    assert names == ["rE_%d_g%d_8_s1" % (rows, cols)], names
    assert len(later_names) == 1 and later_names[0].startswith("E_")
    assert np.array_equal(h, emb[tok])
    monkeypatch.setenv("MOROK_NO_SIDE_OUTPUTS", "1")
    a2, h2, later2, names2, _ = run()
    monkeypatch.delenv("MOROK_NO_SIDE_OUTPUTS")
    assert len(names2) == 2 and names2[0].startswith("E_")
    assert np.array_equal(a, a2) and np.array_equal(h, h2) and np.array_equal(later, later2)


def test_side_output_is_left_alone_when_it_does_not_fit(T):
    """A lookup of another element size than the row kernel's output (f32 rows under a bf16
    normalisation) and one that another input of the same kernel needs first keep their own kernels."""
    from morok_amd import synth, uop

    emb = synth.normal((50, 1024), 84, 0)
    tok = synth.randint((256,), 84, 1, 50)
    h = T.Tensor.from_numpy(emb).embedding(T.Tensor.from_numpy(tok)).contiguous()
    xn = h.rms_norm(-1, 1e-6).cast(uop.BF16)
    xn.realize()
    assert [k.split("_")[0] for k in xn.kernels()] == ["E", "rE"]
    assert np.array_equal(h.to_numpy(), emb[tok])
    # another input of the row kernel (bf16: not a side output of an f32 row) reads the lookup: it is computed
    # first, the row kernel loads it
    x = emb[tok]
    ref = x / np.sqrt((x.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-6) + 2 * x
    h = T.Tensor.from_numpy(emb).embedding(T.Tensor.from_numpy(tok)).contiguous()
    g = h.try_mul(2.0).cast(uop.BF16).contiguous()
    y = h.rms_norm(-1, 1e-6).try_add(g.cast(uop.F32))
    got = y.to_numpy()
    assert [k.split("_")[0] for k in y.kernels()] == ["E", "E", "rE"] and not y.kernels()[-1].endswith("_s1"), y.kernels()
    g_ref = synth.from_bf16(synth.to_bf16(2 * x))
    np.testing.assert_allclose(got, ref - 2 * x + g_ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(h.to_numpy(), x) and np.array_equal(synth.from_bf16(g.to_numpy()), g_ref)
    # two tensors of the row's own kind: both are written by the one kernel
    h = T.Tensor.from_numpy(emb).embedding(T.Tensor.from_numpy(tok)).contiguous()
    g = h.try_mul(2.0).contiguous()
    y = h.rms_norm(-1, 1e-6).try_add(g)
    got = y.to_numpy()
    assert len(y.kernels()) == 1 and y.kernels()[0].endswith("_s2"), y.kernels()
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(h.to_numpy(), x) and np.array_equal(g.to_numpy(), 2 * x)


@pytest.mark.parametrize("seed", range(12))
def test_random_row_kernels_with_side_outputs(T, seed, monkeypatch):
    """Random elementwise chains with `contiguous()` at random places in front of a row statistic
    (sum or max over the last axis, consumed by the same rows), on small integers so that every value
    is exact: the result and every tensor the caller asked to have in memory equal numpy's, whether
    the row kernel writes them itself or they get kernels of their own, and both ways give the same
    kernels' worth of values."""
    rng = np.random.default_rng(4000 + seed)
    rows, cols = int(rng.choice([128, 256, 300, 512])), int(rng.choice([256, 512, 1024, 2048]))
    if seed % 4 == 3:
        rows = cols = 512                                     # square: one operand is read transposed
    x = rng.integers(-3, 4, size=(rows, cols)).astype(np.float32)

    def build():
        a, t = x, T.Tensor.from_numpy(x)
        kept = []
        r = np.random.default_rng(5000 + seed)
        for _ in range(int(r.integers(1, 4))):
            kind = r.choice(["add", "mul", "neg", "contig", "contig"])
            if kind == "add":
                a, t = a + 2.0, t.try_add(T.Tensor.const(2.0))
            elif kind == "mul":
                a, t = a * 2.0, t.try_mul(T.Tensor.const(2.0))
            elif kind == "neg":
                a, t = -a, t.try_mul(T.Tensor.const(-1.0))
            else:
                a, t = a.copy(), t.contiguous()
                kept.append((a, t))
        a, t = a.copy(), t.contiguous()
        kept.append((a, t))
        if r.integers(0, 2):
            a2, t2 = a * a, t.try_mul(t).contiguous()         # a second tensor of the row's kind, built on the first
            kept.append((a2, t2))
        else:
            a2, t2 = a, t
        if r.integers(0, 2):
            stat_a, stat_t = a2.sum(1, keepdims=True), t2.sum(1, keepdim=True)
        else:
            stat_a, stat_t = a2.max(1, keepdims=True), t2.max(1, keepdim=True)
        if rows == cols:
            ya, yt = a.T + stat_a, t.try_permute([1, 0]).try_add(stat_t)
        else:
            ya, yt = a2 - stat_a + a, t2.try_sub(stat_t).try_add(t)
        return ya, yt, kept

    ya, yt, kept = build()
    got = yt.to_numpy()
    names = list(yt.kernels())
    np.testing.assert_array_equal(got, ya)
    for a, t in kept:
        np.testing.assert_array_equal(t.to_numpy(), a)
    assert names[-1].startswith("rE_"), names
    monkeypatch.setenv("MOROK_NO_SIDE_OUTPUTS", "1")
    ya2, yt2, kept2 = build()
    np.testing.assert_array_equal(yt2.to_numpy(), ya)
    names2 = list(yt2.kernels())
    for a, t in kept2:
        np.testing.assert_array_equal(t.to_numpy(), a)
    monkeypatch.delenv("MOROK_NO_SIDE_OUTPUTS")
    assert len(names) <= len(names2)
    if "_s" in names[-1].split("_g")[-1]:
        assert len(names) < len(names2)                       # every side output saved a kernel


def test_beam_search_over_generated_kernels_keeps_values(T, tmp_path, monkeypatch):
    """Under MOROK_BEAM the choices of generated elementwise and reduce kernels are searched on the
    device (candidates timed on scratch buffers of the real sizes); whatever wins, elementwise
    results are the bits of the heuristic kernel and reductions stay within the reduction
    tolerance of float64; the second realization takes its choices from the disk cache."""
    from morok_amd import synth, uop

    Tensor = T.Tensor
    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)
    x = synth.normal((768, 2048), 61, 0)
    y = synth.normal((768, 2048), 61, 1)
    idx = synth.randint((4096,), 61, 2, 768)

    def graphs():
        tx, ty = Tensor.from_numpy(x), Tensor.from_numpy(y)
        e = tx.try_mul(ty).try_add(tx).cast(uop.BF16)                  # elementwise, bf16 out
        r = tx.try_exp().sum(-1)                                        # 768 wave reductions
        f = tx.try_reshape([3, 512 * 1024]).sum(-1)                     # few outputs, long folds
        g = tx.embedding(Tensor.from_numpy(idx)).try_add(Tensor.from_numpy(y[:1]).try_expand([4096, 2048]))   # gather + broadcast
        return e, r, f, g

    monkeypatch.delenv("MOROK_BEAM", raising=False)
    want = [t.to_numpy() for t in graphs()]
    monkeypatch.setenv("MOROK_BEAM", "2")
    timed_total = 0
    got = []
    for t in graphs():
        got.append(t.to_numpy())
        timed, hits = T.last_beam_search()
        assert hits == 0
        timed_total += timed
    assert timed_total >= 20
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[3], want[3])
    ref_r = np.exp(x.astype(np.float64)).sum(-1)
    assert np.abs(got[1] - ref_r).max() <= 1e-4 * np.abs(ref_r).max()
    ref_f = x.astype(np.float64).reshape(3, -1).sum(-1)
    assert np.abs(got[2] - ref_f).max() <= 1e-4 * np.abs(x).astype(np.float64).reshape(3, -1).sum(-1).max()
    for t, w in zip(graphs(), got):
        assert np.array_equal(t.to_numpy(), w)                          # same choices, same bits
        assert T.last_beam_search()[0] == 0 and T.last_beam_search()[1] >= 1
    # a row-resident kernel under the search: whatever workgroup size wins, rms_norm stays within
    # the f32 tolerance of the unsearched kernel (the row sum changes its order only)
    monkeypatch.delenv("MOROK_BEAM", raising=False)
    base = Tensor.from_numpy(x).rms_norm(-1, 1e-6).to_numpy()
    monkeypatch.setenv("MOROK_BEAM", "2")
    searched = Tensor.from_numpy(x).rms_norm(-1, 1e-6).to_numpy()
    assert T.last_kernels()[0].startswith("rE_768_g2048") and T.last_beam_search()[0] >= 3
    assert np.abs(searched - base).max() <= 1e-5 * np.abs(base).max()


# ---------------------------------------------------------------- flat upcast (odd innermost axes)
@pytest.mark.parametrize("shape,dtype", [((1 << 16, 3), "f32"), ((1000, 333), "bf16"), ((64, 50257 // 7 * 8 + 1), "f32"), ((12, 5, 7, 2), "f32"),
                                         ((4096, 1), "f32")])
def test_flat_upcast_elementwise(T, shape, dtype):
    """An innermost axis that does not divide into whole 16-byte groups (an odd vocabulary, [N, 3]
    points, a column) while the element count does: the kernel walks its output as one flat run,
    operands of the output's own shape are read with vector loads at the flat index, and operands
    seen through movement ops (a broadcast row, a transposed square) keep their coordinates."""
    from morok_amd import synth, uop

    n = int(np.prod(shape))
    if dtype == "bf16":
        xb, yb = synth.normal_bf16(shape, 71, 0), synth.normal_bf16(shape, 71, 1)
        x, y = synth.from_bf16(xb), synth.from_bf16(yb)
        tx, ty = T.Tensor.from_numpy(xb, uop.BF16), T.Tensor.from_numpy(yb, uop.BF16)
        got = synth.from_bf16(tx.try_mul(ty).try_add(tx).to_numpy())
        want = synth.from_bf16(synth.to_bf16(x * y + x))
    else:
        x, y = synth.normal(shape, 71, 0), synth.normal(shape, 71, 1)
        tx, ty = T.Tensor.from_numpy(x), T.Tensor.from_numpy(y)
        got = tx.try_mul(ty).try_add(tx).to_numpy()
        want = x * y + x
    name = T.last_kernels()[0]
    width = 16 // (2 if dtype == "bf16" else 4)
    if shape[-1] % width and n % width == 0:
        assert name.endswith("f") and name.startswith("E_%d_" % n), name       # flat, full width
    if dtype == "f32":
        assert np.array_equal(got, (x * y + x).astype(np.float32)) or np.allclose(got, want, rtol=1e-6, atol=0)
        # a broadcast row stays on coordinates while x is read flat
        row = synth.normal((1,) * (len(shape) - 1) + (shape[-1],), 71, 2)
        got2 = tx.try_add(T.Tensor.from_numpy(row).try_expand(list(shape))).to_numpy()
        assert np.array_equal(got2, x + row)
    else:
        assert np.array_equal(got, want)


def test_flat_upcast_keeps_moved_operands_on_coordinates(T):
    from morok_amd import synth

    x, y = synth.normal((6, 6), 72, 0), synth.normal((6, 6), 72, 1)     # 36 elements: groups of 4, rows of 6
    tx, ty = T.Tensor.from_numpy(x), T.Tensor.from_numpy(y)
    got = tx.try_add(ty.try_permute([1, 0])).to_numpy()                   # same shape, but not the same positions
    assert np.array_equal(got, x + y.T) and T.last_kernels()[0].endswith("f")
    got = tx.try_add(tx.try_permute([1, 0])).to_numpy()                   # the same tensor both ways: no flat read at all
    assert np.array_equal(got, x + x.T) and not T.last_kernels()[0].endswith("f")


@pytest.mark.parametrize("shape", [(256, 192, 128), (100, 40, 72), (512, 512, 256), (64, 64, 64)])
def test_half_precision_matmul_hand_written_and_generated(T, oracle, shape):
    """Tensor::matmul on half operands: the hand-written f16 kernels (gemm_f16: the tiled body around
    v_mfma_f32_16x16x32_f16), and with them switched off the WMMA route (f16 tensor core of the CDNA
    table, f32 accumulate, direct-copy variant where its tiles divide the shape, the padded
    register-staged one elsewhere), as a kernel of its own also in the middle of an expression.
    Both against the oracle, and with the same bits as each other."""
    from morok_amd import synth

    M, N, K = shape
    a = synth.normal((M, K), 91, 0).astype(np.float16)
    b = synth.normal((K, N), 91, 1).astype(np.float16)
    ta, tb = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
    c = ta.matmul(tb)
    hand = c.to_numpy()
    assert c.kernels() == ["gemm_f16_%d_%d_%d" % (M, N, K)] and hand.dtype == np.float16
    ref = oracle.gemm_f16(a, b).astype(np.float64)
    assert np.abs(hand - ref).max() <= 2e-2 * np.abs(ref).max() and np.abs(hand - ref).max() <= 2e-3 * np.abs(ref).max()
    lin = ta.linear(T.Tensor.from_numpy(np.ascontiguousarray(b.T)))      # x @ w.T with w stored [N, K]
    got = lin.to_numpy()
    if K % 8 == 0 and N % 8 == 0:
        assert lin.kernels()[-1].startswith("gemm_f16")
    assert np.abs(got - ref).max() <= 2e-3 * np.abs(ref).max()
    T.set_fusion(False)
    c = ta.matmul(tb)
    got = c.to_numpy()
    assert c.kernels() == ["r_tc_%d_%d_%d" % (M, N, K)] and got.dtype == np.float16
    assert np.array_equal(got.view(np.uint16), hand.view(np.uint16))
    both = ta.matmul(tb).try_add(ta.matmul(tb))
    got2 = both.to_numpy()
    assert sum(k.startswith("r_tc_") for k in both.kernels()) == 2
    assert np.array_equal(got2, (got.astype(np.float32) * 2).astype(np.float16))


# ---------------------------------------------------------------- row-resident kernels with chained reductions
@pytest.mark.parametrize("rows,cols", [(256, 1024), (128, 8192), (1000, 512), (300, 2048)])
def test_generated_softmax_family_is_one_kernel(T, oracle, rows, cols):
    """softmax, log_softmax and a layer norm built from tensor ops are each an elementwise kernel fed
    by two keepdim reductions over the last axis, the second building on the first: with the
    hand-written softmax switched off (or for bf16, which it does not cover) they run as ONE
    row-resident kernel: the row is loaded once, both totals stay in registers."""
    from morok_amd import synth, uop

    x = synth.normal((rows, cols), 95, 0, sigma=2.0)
    T.set_fusion(False)
    t = T.Tensor.from_numpy(x).softmax(-1)
    got = t.to_numpy()
    assert len(t.kernels()) == 1 and t.kernels()[0].startswith("rE_%d_g%d" % (rows, cols)) and t.kernels()[0].endswith("_x2")
    np.testing.assert_allclose(got, oracle.softmax_f32(x), rtol=1e-5, atol=1e-9)
    ls = T.Tensor.from_numpy(x).log_softmax(-1)
    got = ls.to_numpy()
    assert len(ls.kernels()) == 1 and ls.kernels()[0].endswith("_x2")
    x64 = x.astype(np.float64)
    ref = x64 - x64.max(-1, keepdims=True)
    ref = ref - np.log(np.exp(ref).sum(-1, keepdims=True))
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    tx = T.Tensor.from_numpy(x)
    xc = tx.try_sub(tx.mean(-1, keepdim=True))
    ln = xc.try_mul(xc.try_mul(xc).mean(-1, keepdim=True).try_add(T.Tensor.const(1e-5)).try_rsqrt())
    got = ln.to_numpy()
    assert len(ln.kernels()) == 1 and ln.kernels()[0].endswith("_x2")
    c64 = x64 - x64.mean(-1, keepdims=True)
    ref = c64 / np.sqrt((c64 * c64).mean(-1, keepdims=True) + 1e-5)
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
    T.set_fusion(True)
    xb = synth.normal_bf16((rows, cols), 95, 1)
    tb = T.Tensor.from_numpy(xb, uop.BF16).softmax(-1)
    got = synth.from_bf16(tb.to_numpy())
    assert len(tb.kernels()) == 1 and tb.kernels()[0].endswith("_x2")
    ref = oracle.softmax_f32(synth.from_bf16(xb))
    assert np.abs(got - ref).max() <= 2e-2 * ref.max()


def test_chained_row_fusion_falls_back_when_a_total_is_needed_elsewhere(T):
    from morok_amd import synth

    x = synth.normal((256, 1024), 96, 0)
    T.set_fusion(False)
    tx = T.Tensor.from_numpy(x)
    m = tx.max(-1, keepdim=True)
    e = tx.try_sub(m).try_exp()
    both = e.try_div(e.sum(-1, keepdim=True)).try_add(m.try_expand([256, 1024]))     # the maximum has a second reader
    got = both.to_numpy()
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(-1, keepdims=True))
    ref = e64 / e64.sum(-1, keepdims=True) + x64.max(-1, keepdims=True)
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max() and len(both.kernels()) >= 2


def test_row_fusion_is_refused_when_the_reduction_is_read_at_other_rows(T):
    """x[i, j] + rowsum[j] (the row totals transposed), a batch permute of them and a shifted slice
    of them over square shapes: the consumer does not read its own row's total, so these must not
    become the row-resident kernel; values against float64."""
    from morok_amd import synth

    x = synth.normal((256, 256), 97, 0)
    x64 = x.astype(np.float64)
    tx = T.Tensor.from_numpy(x)
    rs = tx.sum(1, keepdim=True)
    same = tx.try_add(rs.try_expand([256, 256]))
    got = same.to_numpy()
    assert same.kernels() == ["rE_256_g256_4"]
    np.testing.assert_allclose(got, x64 + x64.sum(1, keepdims=True), rtol=1e-4, atol=1e-4)
    other = tx.try_add(tx.sum(1, keepdim=True).try_transpose(0, 1).try_expand([256, 256]))
    got = other.to_numpy()
    assert not any(k.startswith("rE_") for k in other.kernels())
    np.testing.assert_allclose(got, x64 + x64.sum(1)[None, :], rtol=1e-4, atol=1e-4)
    b = synth.normal((128, 128, 64), 97, 1)
    b64 = b.astype(np.float64)
    tb = T.Tensor.from_numpy(b)
    sw = tb.try_mul(tb.max(2, keepdim=True).try_permute([1, 0, 2]).try_expand([128, 128, 64]))
    got = sw.to_numpy()
    assert not any(k.startswith("rE_") for k in sw.kernels())
    np.testing.assert_allclose(got, b64 * b64.max(2, keepdims=True).transpose(1, 0, 2), rtol=1e-5, atol=1e-6)
    y = synth.normal((512, 256), 97, 2)
    y64 = y.astype(np.float64)
    ty = T.Tensor.from_numpy(y)
    sh = ty.try_shrink([(0, 256), (0, 256)]).try_add(ty.sum(1, keepdim=True).try_shrink([(256, 512), (0, 1)]).try_expand([256, 256]))
    got = sh.to_numpy()
    np.testing.assert_allclose(got, y64[:256] + y64.sum(1, keepdims=True)[256:], rtol=1e-4, atol=1e-4)
