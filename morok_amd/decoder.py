"""A pre-norm decoder transformer block composed from the lazy tensor API (llama layout:
RMSNorm -> QKV -> RoPE -> causal attention -> O-proj + residual -> RMSNorm -> SwiGLU MLP +
residual).  morok has no decoder-block function of its own; this is the caller-side
composition of its ops (tensor/src/transformer.rs:12-137, tensor/src/nn/norm.rs:92-111,
tensor/src/activation.rs:309-318, tensor/src/matmul.rs:82-110) in bfloat16, with the casts
back to bfloat16 that rms_norm's f32 promotion requires placed at each stage output.
"""
import numpy as np

from . import synth, uop
from .tensor import Tensor

WEIGHT_NAMES = ("emb", "w_an", "Wq", "Wk", "Wv", "Wo", "w_fn", "W1", "W3", "W2")


def rope_tables(seq, dim, theta=10000.0):
    """cos/sin [seq, dim/2] in f32: angle(p, i) = p * theta^(-2i/dim)."""
    inv = (theta ** (-np.arange(0, dim, 2, dtype=np.float64) / dim))
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def synthetic_weights(hidden, ffn, vocab, seed=0):
    """Random-init bf16 weights (uint16 bit patterns), scaled so that activations stay O(1)."""
    shapes = {"emb": (vocab, hidden), "w_an": (hidden,), "Wq": (hidden, hidden), "Wk": (hidden, hidden),
              "Wv": (hidden, hidden), "Wo": (hidden, hidden), "w_fn": (hidden,), "W1": (hidden, ffn),
              "W3": (hidden, ffn), "W2": (ffn, hidden)}
    w = {}
    for tid, name in enumerate(WEIGHT_NAMES):
        shp = shapes[name]
        if len(shp) == 1:
            vals = 1.0 + synth.normal(shp, seed, 100 + tid, sigma=0.1)
        else:
            vals = synth.normal(shp, seed, 100 + tid, sigma=1.0 if name == "emb" else 1.0 / np.sqrt(shp[0]))
        w[name] = synth.to_bf16(vals)
    return w


class DecoderBlock:
    """Holds the device-resident weights and builds the lazy graph of one forward pass."""

    def __init__(self, weights, batch, seq, hidden, heads, ffn, eps=1e-6, theta=10000.0, device_id=0,
                 fuse_projections=True, linear_layout=False):
        """fuse_projections: store Wq|Wk|Wv and W1|W3 side by side and run each group as one
        product (same dot products, so the same bits): one launch instead of three / two, and the
        gate+up product at hidden 4096 / ffn 11008 fills whole rounds of output tiles over the
        compute units where two separate products each leave the last round two thirds empty.
        linear_layout: hold every projection as `nn::Linear` does, [out_features, in_features]
        (tensor/src/nn/linear.rs:9-14), and multiply with `linear` (x @ w.T): the same dot products; the kernels
        read the weight in place, and a handful of tokens stream it once."""
        assert hidden % heads == 0
        self.batch, self.seq, self.hidden, self.heads, self.ffn, self.eps = batch, seq, hidden, heads, ffn, eps
        self.dim = hidden // heads
        self.linear_layout = bool(linear_layout)
        projections = ("Wq", "Wk", "Wv", "Wo", "W1", "W2", "W3")
        stored = {k: (np.ascontiguousarray(weights[k].T) if self.linear_layout and k in projections else np.ascontiguousarray(weights[k]))
                  for k in WEIGHT_NAMES}
        self.w = {k: Tensor.from_numpy(stored[k], uop.BF16, device_id) for k in WEIGHT_NAMES}
        self.fused = bool(fuse_projections)
        if self.fused:
            axis = 0 if self.linear_layout else 1
            self.w["Wqkv"] = Tensor.cat([self.w["Wq"], self.w["Wk"], self.w["Wv"]], axis).realize()
            self.w["W13"] = Tensor.cat([self.w["W1"], self.w["W3"]], axis).realize()
        cos, sin = rope_tables(seq, self.dim, theta)
        self.cos_host, self.sin_host = cos, sin
        self.cos = Tensor.from_numpy(cos.reshape(1, 1, seq, self.dim // 2), device_id=device_id)
        self.sin = Tensor.from_numpy(sin.reshape(1, 1, seq, self.dim // 2), device_id=device_id)
        # the same tables shaped for a token-major [batch, seq, heads, dim] operand
        self.cos_tm = Tensor.from_numpy(cos.reshape(1, seq, 1, self.dim // 2), device_id=device_id)
        self.sin_tm = Tensor.from_numpy(sin.reshape(1, seq, 1, self.dim // 2), device_id=device_id)

    def _heads(self, x):
        """[T, hidden] token-major -> [B, H, S, D] head-major (a view: no copy by itself)."""
        return x.try_reshape([self.batch, self.seq, self.heads, self.dim]).try_permute([0, 2, 1, 3])

    def _proj(self, x, name):
        """x @ W for the projection `name`, in whichever layout the block holds it."""
        return x.linear(self.w[name]) if self.linear_layout else x.matmul(self.w[name])

    def _norm(self, x, weight):
        return x.rms_norm(-1, self.eps).try_mul(weight).cast(uop.BF16)

    def forward(self, tokens, with_cache=False):
        """tokens: int32 Tensor [batch*seq].  Returns the lazy bf16 [batch*seq, hidden] output; with_cache: also the
        rotated keys and the values as [batch, heads, seq, dim] tensors (what `decode_step` takes as its past)."""
        w, T = self.w, self.batch * self.seq
        h = w["emb"].embedding(tokens).contiguous()
        xn = self._norm(h, w["w_an"])
        if self.fused:
            qkv = self._proj(xn, "Wqkv")
            xv = qkv.try_shrink([(0, T), (2 * self.hidden, 3 * self.hidden)])
            # q and k lie side by side in the packed product: one rotary kernel over 2 * heads heads
            # (the same per-head arithmetic).  Its result stays token-major (whole 2 * hidden rows
            # in, whole rows out); q and k are head-major views of its two halves, which the
            # attention kernel reads in place
            xqk = qkv.try_shrink([(0, T), (0, 2 * self.hidden)])
            qk = xqk.try_reshape([self.batch, self.seq, 2 * self.heads, self.dim])
            qk = qk.apply_rotary_emb(self.cos_tm, self.sin_tm, False).cast(uop.BF16).contiguous()
            full = [(0, self.batch), (0, self.seq), None, (0, self.dim)]
            q = qk.try_shrink([r if r else (0, self.heads) for r in full]).try_permute([0, 2, 1, 3])
            k = qk.try_shrink([r if r else (self.heads, 2 * self.heads) for r in full]).try_permute([0, 2, 1, 3])
        else:
            xq, xk, xv = self._proj(xn, "Wq"), self._proj(xn, "Wk"), self._proj(xn, "Wv")
            q = self._heads(xq).apply_rotary_emb(self.cos, self.sin, False).cast(uop.BF16)
            k = self._heads(xk).apply_rotary_emb(self.cos, self.sin, False).cast(uop.BF16)
        v = self._heads(xv)
        a = q.scaled_dot_product_attention(k, v, is_causal=True)
        a = a.try_permute([0, 2, 1, 3]).try_reshape([T, self.hidden])
        h2 = h.try_add(self._proj(a, "Wo")).contiguous()
        xn2 = self._norm(h2, w["w_fn"])
        if self.fused:
            gu = self._proj(xn2, "W13")
            g = gu.try_shrink([(0, T), (0, self.ffn)]).silu().try_mul(gu.try_shrink([(0, T), (self.ffn, 2 * self.ffn)]))
        else:
            g = self._proj(xn2, "W1").silu().try_mul(self._proj(xn2, "W3"))
        out = h2.try_add(self._proj(g, "W2"))
        return (out, k.contiguous(), v.contiguous()) if with_cache else out

    def decode_step(self, tokens, past_k, past_v, pos):
        """One new token per sequence against the keys and values of the `pos` tokens before it, the way the reference
        carries a cache through its attention operator (onnx/src/registry/transformer.rs:74-75: K = cat(past, new) along
        the sequence axis, then scaled_dot_product_attention): tokens int32 [batch], past_k / past_v bf16
        [batch, heads, pos, dim] (keys already rotated), pos the new token's position.  Returns the lazy
        (output [batch, hidden], keys [batch, heads, pos + 1, dim], values): the row a causal forward pass over
        pos + 1 tokens would give for the last token.  With Linear-layout weights the projections stream their weights
        once, and the attention is one query per head over pos + 1 keys."""
        assert self.fused, "decode_step uses the packed projections"
        w, B, H, D = self.w, self.batch, self.heads, self.dim
        cos, sin = rope_tables(pos + 1, D)
        cos_p = Tensor.from_numpy(np.ascontiguousarray(cos[pos].reshape(1, 1, 1, D // 2)))
        sin_p = Tensor.from_numpy(np.ascontiguousarray(sin[pos].reshape(1, 1, 1, D // 2)))
        h = w["emb"].embedding(tokens).contiguous()
        xn = self._norm(h, w["w_an"])
        qkv = self._proj(xn, "Wqkv")
        xv = qkv.try_shrink([(0, B), (2 * self.hidden, 3 * self.hidden)])
        qk = qkv.try_shrink([(0, B), (0, 2 * self.hidden)]).try_reshape([B, 1, 2 * H, D])
        qk = qk.apply_rotary_emb(cos_p, sin_p, False).cast(uop.BF16).contiguous()
        q = qk.try_shrink([(0, B), (0, 1), (0, H), (0, D)]).try_permute([0, 2, 1, 3])
        k_new = qk.try_shrink([(0, B), (0, 1), (H, 2 * H), (0, D)]).try_permute([0, 2, 1, 3])
        v_new = xv.try_reshape([B, 1, H, D]).try_permute([0, 2, 1, 3])
        k_all = Tensor.cat([past_k, k_new], 2).contiguous()
        v_all = Tensor.cat([past_v, v_new], 2).contiguous()
        a = q.scaled_dot_product_attention(k_all, v_all)
        a = a.try_permute([0, 2, 1, 3]).try_reshape([B, self.hidden])
        h2 = h.try_add(self._proj(a, "Wo")).contiguous()
        xn2 = self._norm(h2, w["w_fn"])
        gu = self._proj(xn2, "W13")
        g = gu.try_shrink([(0, B), (0, self.ffn)]).silu().try_mul(gu.try_shrink([(0, B), (self.ffn, 2 * self.ffn)]))
        return h2.try_add(self._proj(g, "W2")), k_all, v_all
