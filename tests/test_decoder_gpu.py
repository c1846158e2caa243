"""Decoder transformer block composed from the lazy tensor API, against the CPU oracle's
stage-by-stage restatement (bf16 storage, f32 math, one rounding per stage output)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def run_block(cfg, tokens, weights, fused=True, linear_layout=False):
    from morok_amd import decoder, tensor, uop

    blk = decoder.DecoderBlock(weights, cfg["batch"], cfg["seq"], cfg["hidden"], cfg["heads"], cfg["ffn"], cfg["eps"],
                               fuse_projections=fused, linear_layout=linear_layout)
    out = blk.forward(tensor.Tensor.from_numpy(tokens.astype(np.int32)))
    out.realize()
    return blk, out, out.kernels()


def rel_err(got_bits, ref_bits):
    from morok_amd import synth

    got, ref = synth.from_bf16(got_bits), synth.from_bf16(ref_bits)
    return float(np.abs(got - ref).max() / np.abs(ref).max())


@pytest.mark.parametrize("cfg", [
    dict(batch=2, seq=128, hidden=256, heads=2, ffn=512, vocab=1000, eps=1e-6),
    dict(batch=1, seq=192, hidden=512, heads=4, ffn=1280, vocab=777, eps=1e-6),
    dict(batch=1, seq=256, hidden=4096, heads=32, ffn=11008, vocab=32000, eps=1e-6),
], ids=["h256", "h512", "h4096_seq256"])
def test_decoder_block_vs_oracle(dev, oracle, cfg):
    from morok_amd import decoder, synth

    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=3)
    T = cfg["batch"] * cfg["seq"]
    tok = synth.randint((T,), 3, 1, cfg["vocab"])
    blk, out, kernels = run_block(cfg, tok, w)
    got = out.to_numpy()
    ref = oracle.decoder_block_bf16(tok, w, blk.cos_host, blk.sin_host, cfg["batch"], cfg["seq"], cfg["hidden"],
                                    cfg["heads"], cfg["ffn"], cfg["eps"])
    assert got.shape == ref.shape == (T, cfg["hidden"])
    assert rel_err(got, ref) <= 2e-2   # bf16 GEMM/attention tolerance
    # the matmuls (Wq|Wk|Wv and W1|W3 each as one product) and the attention run as the
    # hand-written kernels
    assert sum(k.startswith("gemm_bf16") for k in kernels) == 4
    assert sum(k.startswith("flash_fwd") for k in kernels) == 1
    assert sum(k.startswith("gemm_bf16_swiglu") for k in kernels) == 1   # silu(gate) * up in the W1|W3 epilogue
    # Seven separate products compute the same dot products.  The gate differs in one place: the
    # epilogue of the packed W1|W3 product takes its reciprocal with the hardware approximation
    # (1 ulp) where the generated elementwise kernel divides exactly, so a small fraction of the
    # gated activations round to the neighbouring bf16 value (and a product with few rows may be
    # spread along K in one layout and not in the other): single roundings falling the other way.
    _, out7, kernels7 = run_block(cfg, tok, w, fused=False)
    assert sum(k.startswith("gemm_bf16") for k in kernels7) == 7
    assert rel_err(out7.to_numpy(), got) <= 1e-2
    assert rel_err(out7.to_numpy(), ref) <= 2e-2


@pytest.mark.parametrize("cfg", [
    dict(batch=2, seq=8, hidden=4096, heads=32, ffn=11008, vocab=32000, eps=1e-6),
    dict(batch=1, seq=40, hidden=1024, heads=8, ffn=2816, vocab=500, eps=1e-6),
    dict(batch=5, seq=1, hidden=256, heads=2, ffn=512, vocab=300, eps=1e-6),      # one position per sequence: every stride of the sequence axis is moot
], ids=["h4096_16tokens", "h1024_40tokens", "h256_seq1"])
def test_decoder_block_few_tokens(dev, oracle, cfg):
    """A handful of tokens: every product has few output tiles against a long K, so it is spread along K (or
    streamed) instead of run as one pass of tiles.  The gate and the rotary embedding, whose fused forms exist for
    the tiled kernels only, run as generated kernels; the residual adds join where the products' results are written."""
    from morok_amd import decoder, synth

    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=4)
    T = cfg["batch"] * cfg["seq"]
    tok = synth.randint((T,), 4, 1, cfg["vocab"])
    blk, out, kernels = run_block(cfg, tok, w)
    got = out.to_numpy()
    ref = oracle.decoder_block_bf16(tok, w, blk.cos_host, blk.sin_host, cfg["batch"], cfg["seq"], cfg["hidden"],
                                    cfg["heads"], cfg["ffn"], cfg["eps"])
    assert rel_err(got, ref) <= 2e-2
    assert sum(k.startswith("gemm_bf16") for k in kernels) == 4
    assert sum(k.startswith("flash_fwd") for k in kernels) == 1
    assert not any(tag in k for k in kernels for tag in ("swiglu", "rope")), kernels
    assert sum("residual" in k for k in kernels) == 2, kernels


@pytest.mark.parametrize("cfg", [
    dict(batch=1, seq=256, hidden=4096, heads=32, ffn=11008, vocab=32000, eps=1e-6),
    dict(batch=2, seq=8, hidden=4096, heads=32, ffn=11008, vocab=32000, eps=1e-6),
    dict(batch=3, seq=1, hidden=512, heads=4, ffn=1280, vocab=777, eps=1e-6),
], ids=["h4096_seq256", "h4096_16tokens", "h512_seq1"])
def test_decoder_block_with_linear_layout_weights(dev, oracle, cfg):
    """Every projection held as nn::Linear holds it ([out_features, in_features], tensor/src/nn/linear.rs:9-14)
    and applied with `linear`: the kernels read the weights in place.  A prefill-sized run keeps the fused
    epilogues (rotary, residual, gate) and gives the bits of the [K, N] block (the same products in the same
    order); a handful of tokens streams every weight once, with the residual adds and the gate inside the streaming kernels."""
    from morok_amd import decoder, synth

    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=6)
    T = cfg["batch"] * cfg["seq"]
    tok = synth.randint((T,), 6, 1, cfg["vocab"])
    blk, out, kernels = run_block(cfg, tok, w, linear_layout=True)
    got = out.to_numpy()
    ref = oracle.decoder_block_bf16(tok, w, blk.cos_host, blk.sin_host, cfg["batch"], cfg["seq"], cfg["hidden"],
                                    cfg["heads"], cfg["ffn"], cfg["eps"])
    assert rel_err(got, ref) <= 2e-2
    products = [k for k in kernels if k.startswith("gemm_bf16")]
    assert len(products) == 4 and all(k.startswith("gemm_bf16_nt") for k in products), kernels
    if T >= 256:
        assert any("rope" in k for k in products) and any("swiglu" in k for k in products), kernels
        _, out_kn, _ = run_block(cfg, tok, w)
        assert np.array_equal(got, out_kn.to_numpy())
    else:
        assert sum("residual" in k for k in products) == 2 and sum("swiglu" in k for k in products) == 1, kernels
        assert not any("rope" in k for k in products), kernels


def test_decoder_block_full_size_properties(dev):
    """hidden 4096, 32 heads, SwiGLU 11008, batch 4 x seq 2048: too large for the CPU oracle in
    a test, so checked through properties that hold at any size: determinism, independence of
    batch entries, and causality (outputs before position p ignore tokens from p on)."""
    from morok_amd import decoder, synth

    cfg = dict(batch=4, seq=2048, hidden=4096, heads=32, ffn=11008, vocab=32000, eps=1e-6)
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=5)
    T = cfg["batch"] * cfg["seq"]
    tok = synth.randint((T,), 5, 1, cfg["vocab"])
    _, out, kernels = run_block(cfg, tok, w)
    a = out.to_numpy()
    assert np.isfinite(synth.from_bf16(a)).all()
    _, out2, _ = run_block(cfg, tok, w)
    assert np.array_equal(a, out2.to_numpy())                       # deterministic
    p = 1500
    tok2 = tok.copy().reshape(cfg["batch"], cfg["seq"])
    tok2[1, p:] = (tok2[1, p:] + 17) % cfg["vocab"]                 # change the tail of sequence 1
    _, out3, _ = run_block(cfg, tok2.reshape(-1), w)
    b = out3.to_numpy().reshape(cfg["batch"], cfg["seq"], -1)
    a4 = a.reshape(cfg["batch"], cfg["seq"], -1)
    assert np.array_equal(a4[0], b[0]) and np.array_equal(a4[2:], b[2:])   # other sequences untouched
    assert np.array_equal(a4[1, :p], b[1, :p])                              # causal prefix untouched
    assert not np.array_equal(a4[1, p:], b[1, p:])
    # one sequence alone gives the same rows as inside the batch
    cfg1 = dict(cfg, batch=1)
    _, out4, _ = run_block(cfg1, tok[: cfg["seq"]], w)
    assert np.array_equal(out4.to_numpy(), a4[0])


def test_memory_planner_on_and_off_give_the_same_bits_in_less_memory(dev, oracle, monkeypatch):
    """tensor/src/memory_planner.rs:1-45 on the device: the decoder block with the planner
    (intermediates share blocks by liveness) and without it (MOROK_NO_MEMORY_PLANNER=1, every
    intermediate keeps a block of its own) must give identical bits, the planned run must reuse
    blocks and hold strictly fewer intermediate bytes, and both must match the oracle."""
    from morok_amd import decoder, synth, tensor

    cfg = dict(batch=1, seq=192, hidden=512, heads=4, ffn=1280, vocab=777, eps=1e-6)
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=3)
    tok = synth.randint((cfg["batch"] * cfg["seq"],), 3, 1, cfg["vocab"])
    monkeypatch.delenv("MOROK_NO_MEMORY_PLANNER", raising=False)
    blk, out, kernels = run_block(cfg, tok, w)
    planned = out.to_numpy()
    reused, saved = tensor.last_memory_plan()
    planned_bytes = tensor.last_intermediate_bytes()
    assert reused >= 2 and saved > 0 and planned_bytes > 0
    monkeypatch.setenv("MOROK_NO_MEMORY_PLANNER", "1")
    _, out2, kernels2 = run_block(cfg, tok, w)
    unplanned = out2.to_numpy()
    assert tensor.last_memory_plan() == (0, 0)
    unplanned_bytes = tensor.last_intermediate_bytes()
    assert kernels2 == kernels
    assert np.array_equal(planned, unplanned)
    assert planned_bytes < unplanned_bytes and unplanned_bytes - planned_bytes == saved
    ref = oracle.decoder_block_bf16(tok, w, blk.cos_host, blk.sin_host, cfg["batch"], cfg["seq"], cfg["hidden"],
                                    cfg["heads"], cfg["ffn"], cfg["eps"])
    assert rel_err(planned, ref) <= 2e-2
    # a block really is shared: run again with the planner and poison nothing -- the second
    # planned run reuses the cached blocks of the first and still gives the same bits
    monkeypatch.delenv("MOROK_NO_MEMORY_PLANNER")
    _, out3, _ = run_block(cfg, tok, w)
    assert np.array_equal(out3.to_numpy(), planned)


@pytest.mark.parametrize("cfg,linear_layout", [
    (dict(batch=2, seq=300, hidden=512, heads=4, ffn=1280, vocab=777, eps=1e-6), True),
    (dict(batch=1, seq=600, hidden=1024, heads=8, ffn=2816, vocab=500, eps=1e-6), False),
    (dict(batch=4, seq=1100, hidden=256, heads=2, ffn=512, vocab=300, eps=1e-6), True),
], ids=["h512_299past", "h1024_599past", "h256_1099past"])
def test_decode_step_over_cached_keys_is_the_last_row_of_a_causal_pass(dev, oracle, cfg, linear_layout):
    """One new token against the cached keys and values of the tokens before it (K = cat(past, new), then attention with
    one query per head, as the reference's attention operator carries its past: onnx/src/registry/transformer.rs:74-75)
    gives the row a causal pass over the whole sequence gives for its last token: against the oracle's block over all
    tokens, and against this library's own full pass.  The attention of the step is the kernel that streams the keys."""
    from morok_amd import decoder, synth, tensor

    B, S = cfg["batch"], cfg["seq"]
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=8)
    tok = synth.randint((B * S,), 8, 1, cfg["vocab"]).reshape(B, S)
    # the whole sequence, causal
    full_cfg = dict(cfg)
    blk, out, _ = run_block(full_cfg, tok.reshape(-1), w, linear_layout=linear_layout)
    full = out.to_numpy().reshape(B, S, cfg["hidden"])
    ref = oracle.decoder_block_bf16(tok.reshape(-1), w, blk.cos_host, blk.sin_host, B, S, cfg["hidden"], cfg["heads"], cfg["ffn"],
                                    cfg["eps"]).reshape(B, S, cfg["hidden"])
    # the first S - 1 tokens, keeping their keys and values
    P = S - 1
    pre = decoder.DecoderBlock(w, B, P, cfg["hidden"], cfg["heads"], cfg["ffn"], cfg["eps"], linear_layout=linear_layout)
    o, k, v = pre.forward(tensor.Tensor.from_numpy(np.ascontiguousarray(tok[:, :P]).reshape(-1).astype(np.int32)), with_cache=True)
    o.realize(), k.realize(), v.realize()
    assert tuple(k.shape) == (B, cfg["heads"], P, cfg["hidden"] // cfg["heads"])
    # the last token against that cache
    step = decoder.DecoderBlock(w, B, 1, cfg["hidden"], cfg["heads"], cfg["ffn"], cfg["eps"], linear_layout=linear_layout)
    y, k_all, v_all = step.decode_step(tensor.Tensor.from_numpy(np.ascontiguousarray(tok[:, P]).astype(np.int32)), k, v, P)
    y.realize()
    kernels = y.kernels()
    got = y.to_numpy()
    assert got.shape == (B, cfg["hidden"])
    assert rel_err(got, ref[:, P]) <= 2e-2
    assert rel_err(got, full[:, P]) <= 2e-2
    att = [n for n in kernels if n.startswith("flash_fwd")]
    assert len(att) == 1 and ("_%d_1_%d" % (B * cfg["heads"], S)) in att[0], kernels   # one query per head over S keys
    # the cache the step hands on: the past with the new token's key and value appended
    ka, va = k_all.to_numpy(), v_all.to_numpy()
    assert ka.shape == (B, cfg["heads"], S, cfg["hidden"] // cfg["heads"])
    assert np.array_equal(ka[:, :, :P], k.to_numpy()) and np.array_equal(va[:, :, :P], v.to_numpy())
