"""Randomised differential tests of the fused kernels against their unfused counterparts on
the GPU: attention over random strided layouts against the kernel over dense copies (bit for
bit, padding between rows untouched), the GEMM residual epilogue against product-then-add (bit
for bit), and the generated tensor-core kernel over random tile choices and padded shapes
against float64.  Seeds are fixed; every case is small."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, sched, synth, uop as U

pytestmark = pytest.mark.gpu
D = 128
NAN = np.uint16(0x7FC0)


def _layout(rng, t):
    """`t` [B, H, S, D] stored with a random order of its first three axes and random padding
    behind each row; returns the padded array and the (batch, head, row) element strides."""
    perm = [int(p) for p in rng.permutation(3)]
    pad = int(rng.integers(0, 3)) * 8
    big = np.full([t.shape[i] for i in perm] + [D + pad], NAN, np.uint16)
    big[..., :D] = t.transpose(perm + [3])
    strides = [0, 0, 0]
    for pos, ax in enumerate(perm):
        strides[ax] = big.strides[pos] // 2
    return big, strides


@pytest.mark.parametrize("seed", range(16))
def test_attention_over_random_layouts(dev, seed):
    rng = np.random.default_rng(7100 + seed)
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    Sq, Sk = int(rng.integers(1, 400)), int(rng.integers(1, 400))
    causal = bool(rng.integers(0, 2))
    if causal:
        Sk = Sq
    q, k, v = (synth.normal_bf16((B, H, s, D), 7100 + seed, i) for i, s in enumerate((Sq, Sk, Sk)))
    bq, bk, bv = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (q, k, v))
    bo = dev.buffer(q.nbytes)
    scale = 1 / np.sqrt(D)
    ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, Sq, Sk, D, scale, causal, dev.device_id)
    want = bo.copyout(np.uint16, q.shape)
    (qb, qs), (kb, ks), (vb, vs) = (_layout(rng, t) for t in (q, k, v))
    ob, os_ = _layout(rng, np.zeros_like(q))
    ob[...] = NAN
    bufs = [morok_amd.Buffer.from_numpy(x, dev.device_id) for x in (qb, kb, vb, ob)]
    ops.flash_attn_fwd_bf16_strided(bufs[0], bufs[1], bufs[2], bufs[3], B, H, Sq, Sk, D, scale, qs + ks + vs + os_,
                                    (0, 0, 0, 0), causal, dev.device_id)
    out = bufs[3].copyout(np.uint16, ob.shape)
    assert np.all(out[..., D:] == NAN)                         # nothing written between the rows
    idx = np.indices((B, H, Sq))
    offs = idx[0] * os_[0] + idx[1] * os_[1] + idx[2] * os_[2]
    got = out.reshape(-1)[(offs[..., None] + np.arange(D)).reshape(-1)].reshape(B, H, Sq, D)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("seed", range(16))
def test_residual_epilogue_random_shapes(dev, seed):
    rng = np.random.default_rng(7200 + seed)
    M, N, K = int(rng.integers(1, 700)), int(rng.integers(1, 90)) * 8, int(rng.integers(1, 160)) * 8
    a, b, r = (synth.normal_bf16(sh, 7200 + seed, i) for i, sh in enumerate(((M, K), (K, N), (M, N))))
    ba, bb, br = (morok_amd.Buffer.from_numpy(t, dev.device_id) for t in (a, b, r))
    bc, bp = dev.buffer(M * N * 2), dev.buffer(M * N * 2)
    ops.gemm_bf16_residual(ba, bb, br, bc, M, N, K, dev.device_id)
    ops.gemm_bf16(ba, bb, bp, M, N, K, dev.device_id)
    want = synth.to_bf16(synth.from_bf16(bp.copyout(np.uint16, (M, N))) + synth.from_bf16(r))
    assert np.array_equal(bc.copyout(np.uint16, (M, N)), want)


@pytest.mark.parametrize("seed", range(32))
def test_generated_tensor_core_random_choices(dev, seed):
    rng = np.random.default_rng(7300 + seed)
    M, N, K = int(rng.integers(1, 300)), int(rng.integers(1, 40)) * 8, int(rng.integers(1, 40)) * 8
    while True:  # not every combination splits into whole copies per work-item: draw again
        opts = (int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 4, 8])),
                int(rng.choice([0, 1, 2, 4])))
        try:
            kern = sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts)
            break
        except morok_amd.MorokHipError:
            continue
    a, b = synth.normal_bf16((M, K), 7300 + seed, 0), synth.normal_bf16((K, N), 7300 + seed, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)
    bc = morok_amd.Buffer.from_numpy(np.full(M * N + 512, NAN, np.uint16), dev.device_id)
    k = morok_amd.Kernel.get_or_compile(kern, "r_tc_random")
    plan = morok_amd.ExecutionPlan()
    plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(ba), plan.add_buffer(bb)])
    plan.build().execute()
    got = bc.copyout(np.uint16, (M * N + 512,))
    assert np.all(got[M * N:] == NAN)
    c = synth.from_bf16(got[:M * N].reshape(M, N))
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    assert np.all(np.isfinite(c)) and np.abs(c - ref).max() <= 2e-2 * max(np.abs(ref).max(), 1e-6)


@pytest.mark.parametrize("seed", range(24))
def test_generated_tensor_core_direct_copy_random_choices(dev, seed):
    """Random workgroup shapes, tile counts and K depths of the direct-copy variant, both tile
    shapes (16x16x32 and 32x32x16): the bits of the hand-written GEMM (which the register-only
    kernels also produce), nothing written behind the result."""
    rng = np.random.default_rng(7400 + seed)
    tc = int(rng.choice([3, 7]))
    while True:
        opts = (int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 4, 8])), 0,
                2 + seed % 2)   # two stages of both tiles, or a third one of the second operand's
        t = 16 if tc == 3 else 32
        bm, bn = opts[0] * opts[2] * t, opts[1] * opts[3] * t
        M, N, K = bm * int(rng.integers(1, 5)), bn * int(rng.integers(1, 5)), 64 * int(rng.integers(1, 7))
        if M * N > 1 << 21:
            continue
        try:
            kern = sched.build_wmma_matmul_lds_opts(tc, M, N, K, U.BF16, opts)
            break
        except morok_amd.MorokHipError:
            continue
    a, b = synth.normal_bf16((M, K), 7400 + seed, 0), synth.normal_bf16((K, N), 7400 + seed, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)
    bc = morok_amd.Buffer.from_numpy(np.full(M * N + 512, NAN, np.uint16), dev.device_id)
    k = morok_amd.Kernel.get_or_compile(kern, "r_tc_dma_random")
    plan = morok_amd.ExecutionPlan()
    plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(ba), plan.add_buffer(bb)])
    plan.build().execute()
    got = bc.copyout(np.uint16, (M * N + 512,))
    assert np.all(got[M * N:] == NAN)
    bh = dev.buffer(M * N * 2)
    ops.gemm_bf16(ba, bb, bh, M, N, K, dev.device_id, 4)       # the tiled kernel (a handful of rows would otherwise be streamed)
    assert np.array_equal(got[:M * N].reshape(M, N), bh.copyout(np.uint16, (M, N))), (tc, opts, (M, N, K))
