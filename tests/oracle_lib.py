"""ctypes access to the CPU oracle (oracle/libmorok_cpu_oracle.so) - the checker the
parity tests compare the HIP path against.  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_DIR = os.path.join(_ROOT, "oracle")
_SO = os.path.join(_DIR, "libmorok_cpu_oracle.so")


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self):
        if not os.path.exists(_SO):
            subprocess.check_call(["make", "-C", _DIR])
        self.lib = C.CDLL(_SO)
        L = self.lib
        L.orc_thread_count.restype = C.c_int
        L.orc_thread_count.argtypes = [C.c_long, C.c_long, C.c_int]
        L.orc_decoder_block_scratch_elems.restype = C.c_size_t
        L.orc_decoder_block_scratch_elems.argtypes = [C.c_int, C.c_int, C.c_int]
        L.orc_unary_f32.restype = C.c_float
        L.orc_binary_f32.restype = C.c_float
        self.max_threads = min(os.cpu_count() or 1, 16)

    def thread_count(self, total, axis, max_threads=None):
        return self.lib.orc_thread_count(total, axis, max_threads or self.max_threads)

    def matmul_f32(self, a, b, threads=None):
        M, K = a.shape
        K2, N = b.shape
        assert K == K2
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        c = np.empty((M, N), np.float32)
        t = threads or self.thread_count(M * N * K, M)
        self.lib.orc_matmul_f32(_ptr(a), _ptr(b), _ptr(c), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(t))
        return c

    def softmax_f32(self, x, threads=None):
        x = np.ascontiguousarray(x, np.float32)
        rows, cols = x.shape
        y = np.empty_like(x)
        scratch = np.empty(2 * rows, np.float32)
        t = threads or self.thread_count(rows * cols, rows)
        self.lib.orc_softmax_f32(_ptr(x), _ptr(y), _ptr(scratch), C.c_long(rows), C.c_long(cols), C.c_int(t))
        return y

    def gemm_bf16(self, a, b, literal=False, threads=None):
        M, K = a.shape
        K2, N = b.shape
        assert K == K2 and a.dtype == np.uint16 and b.dtype == np.uint16
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        c = np.empty((M, N), np.uint16)
        t = threads or self.thread_count(M * N * K, M)
        self.lib.orc_gemm_bf16(_ptr(a), _ptr(b), _ptr(c), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(int(literal)),
                               C.c_int(t))
        return c

    def gemm_f16(self, a, b, threads=None):
        """a [M, K], b [K, N] numpy float16 -> float16 [M, N] (f32 accumulate along k, one rounding)."""
        M, K = a.shape
        N = b.shape[1]
        a, b = np.ascontiguousarray(a, np.float16), np.ascontiguousarray(b, np.float16)
        c = np.empty((M, N), np.float16)
        self.lib.orc_gemm_f16(_ptr(a), _ptr(b), _ptr(c), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(threads or self.max_threads))
        return c

    def sdpa_bf16(self, q, k, v, scale, causal=True, policy=0, threads=None):
        B, H, Sq, D = q.shape
        Sk = k.shape[2]
        q, k, v = (np.ascontiguousarray(t_) for t_ in (q, k, v))
        o = np.empty_like(q)
        self.lib.orc_sdpa_bf16(_ptr(q), _ptr(k), _ptr(v), _ptr(o), C.c_int(B * H), C.c_int(Sq), C.c_int(Sk),
                               C.c_int(D), C.c_float(scale), C.c_int(int(causal)), C.c_int(policy),
                               C.c_int(threads or self.max_threads))
        return o

    def sdpa_bf16_ex(self, q, k, v, scale, causal=False, mask=None, softcap=0.0, threads=None):
        """attn_mask (bool or bf16-as-uint16 array broadcastable to [B, H, Sq, Sk] with the key axis
        full) and softcap, in the reference's order (tensor/src/transformer.rs:96-132)."""
        B, H, Sq, D = q.shape
        Sk = k.shape[2]
        q, k, v = (np.ascontiguousarray(t_) for t_ in (q, k, v))
        o = np.empty_like(q)
        kind, mptr, strides = 0, None, (C.c_long * 3)(0, 0, 0)
        if mask is not None:
            mask = np.ascontiguousarray(mask)
            kind = 1 if mask.dtype == np.bool_ else 2
            assert kind == 1 or mask.dtype == np.uint16
            shape = (1,) * (4 - mask.ndim) + mask.shape
            assert shape[3] == Sk and all(s_ in (1, full) for s_, full in zip(shape[:3], (B, H, Sq)))
            dense = [shape[1] * shape[2] * shape[3], shape[2] * shape[3], shape[3]]
            strides = (C.c_long * 3)(*[0 if shape[i] == 1 else dense[i] for i in range(3)])
            mptr = _ptr(mask.view(np.uint8) if kind == 1 else mask)
        self.lib.orc_sdpa_bf16_ex(_ptr(q), _ptr(k), _ptr(v), _ptr(o), C.c_int(B), C.c_int(H), C.c_int(Sq), C.c_int(Sk),
                                  C.c_int(D), C.c_float(scale), C.c_int(int(causal)), mptr, C.c_int(kind), strides,
                                  C.c_float(softcap), C.c_int(threads or self.max_threads))
        return o

    def sdpa_bf16_rows(self, q, k, v, scale, causal=True, threads=None):
        Sq, D = q.shape
        Sk = k.shape[0]
        q, k, v = (np.ascontiguousarray(t_) for t_ in (q, k, v))
        o = np.empty_like(q)
        self.lib.orc_sdpa_bf16_rows(_ptr(q), _ptr(k), _ptr(v), _ptr(o), C.c_int(Sq), C.c_int(Sk), C.c_int(D),
                                    C.c_float(scale), C.c_int(int(causal)), C.c_int(0),
                                    C.c_int(threads or self.max_threads))
        return o

    def sdpa_f32(self, q, k, v, scale, causal=False, threads=None):
        B, H, Sq, D = q.shape
        Sk = k.shape[2]
        q, k, v = (np.ascontiguousarray(t_, np.float32) for t_ in (q, k, v))
        o = np.empty_like(q)
        self.lib.orc_sdpa_f32(_ptr(q), _ptr(k), _ptr(v), _ptr(o), C.c_int(B * H), C.c_int(Sq), C.c_int(Sk),
                              C.c_int(D), C.c_float(scale), C.c_int(int(causal)), C.c_int(threads or self.max_threads))
        return o

    def rms_norm_f32(self, x, eps):
        x = np.ascontiguousarray(x, np.float32)
        rows, cols = x.reshape(-1, x.shape[-1]).shape
        y = np.empty_like(x)
        self.lib.orc_rms_norm_f32(_ptr(x), _ptr(y), C.c_long(rows), C.c_long(cols), C.c_float(eps))
        return y

    def rms_norm_weight_bf16(self, x, w, eps):
        x = np.ascontiguousarray(x)
        w = np.ascontiguousarray(w)
        rows, cols = x.shape
        y = np.empty_like(x)
        self.lib.orc_rms_norm_weight_bf16(_ptr(x), _ptr(w), _ptr(y), C.c_long(rows), C.c_long(cols), C.c_float(eps))
        return y

    def rope_f32(self, x, cos, sin, interleaved):
        x = np.ascontiguousarray(x, np.float32)
        dim = x.shape[-1]
        rows = x.size // dim
        cos = np.ascontiguousarray(np.broadcast_to(cos, x.shape[:-1] + (dim // 2,)), np.float32)
        sin = np.ascontiguousarray(np.broadcast_to(sin, x.shape[:-1] + (dim // 2,)), np.float32)
        y = np.empty_like(x)
        self.lib.orc_rope_f32(_ptr(x), _ptr(cos), _ptr(sin), _ptr(y), C.c_long(rows), C.c_int(dim),
                              C.c_int(int(interleaved)))
        return y

    def rope_heads_bf16(self, x, cos, sin, batch, seq, heads, dim, apply=True):
        x = np.ascontiguousarray(x)
        cos = np.ascontiguousarray(cos, np.float32)
        sin = np.ascontiguousarray(sin, np.float32)
        y = np.empty((batch, heads, seq, dim), np.uint16)
        self.lib.orc_rope_heads_bf16(_ptr(x), _ptr(cos), _ptr(sin), _ptr(y), C.c_int(batch), C.c_int(seq),
                                     C.c_int(heads), C.c_int(dim), C.c_int(int(apply)))
        return y

    def embedding(self, weight, idx):
        weight = np.ascontiguousarray(weight)
        idx = np.ascontiguousarray(idx, np.int32)
        dim = weight.shape[1]
        out = np.empty(idx.shape + (dim,), weight.dtype)
        fn = self.lib.orc_embedding_f32 if weight.dtype == np.float32 else self.lib.orc_embedding_u16
        fn(_ptr(weight), _ptr(idx), _ptr(out), C.c_long(idx.size), C.c_long(dim))
        return out

    def silu_f32(self, x):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        self.lib.orc_silu_f32(_ptr(x), _ptr(y), C.c_long(x.size))
        return y

    def silu_mul_bf16(self, g, u):
        g = np.ascontiguousarray(g)
        u = np.ascontiguousarray(u)
        y = np.empty_like(g)
        self.lib.orc_silu_mul_bf16(_ptr(g), _ptr(u), _ptr(y), C.c_long(g.size))
        return y

    def add_bf16(self, a, b):
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        y = np.empty_like(a)
        self.lib.orc_add_bf16(_ptr(a), _ptr(b), _ptr(y), C.c_long(a.size))
        return y

    def fp8_to_f32(self, kind, x):
        """kind 0 = E4M3, 1 = E5M2; x: uint8 codes."""
        x = np.ascontiguousarray(x, np.uint8)
        y = np.empty(x.shape, np.float32)
        self.lib.orc_fp8_to_f32(C.c_int(kind), _ptr(x), C.c_long(x.size), _ptr(y))
        return y

    def matmul_fp8_f32(self, kind, a, b):
        a = np.ascontiguousarray(a, np.uint8)
        b = np.ascontiguousarray(b, np.uint8)
        c = np.empty((a.shape[0], b.shape[1]), np.float32)
        self.lib.orc_matmul_fp8_f32(C.c_int(kind), _ptr(a), _ptr(b), _ptr(c), a.shape[0], b.shape[1], a.shape[1])
        return c

    def decoder_block_bf16(self, tok, w, cos, sin, batch, seq, hidden, heads, ffn, eps, threads=None):
        T = batch * seq
        n = self.lib.orc_decoder_block_scratch_elems(T, hidden, ffn)
        work = np.empty(n, np.uint16)
        out = np.empty((T, hidden), np.uint16)
        tok = np.ascontiguousarray(tok, np.int32)
        cos = np.ascontiguousarray(cos, np.float32)
        sin = np.ascontiguousarray(sin, np.float32)
        ws = [np.ascontiguousarray(w[k]) for k in ("emb", "w_an", "Wq", "Wk", "Wv", "Wo", "w_fn", "W1", "W3", "W2")]
        self.lib.orc_decoder_block_bf16(_ptr(tok), *[_ptr(a) for a in ws], _ptr(cos), _ptr(sin), _ptr(out),
                                        _ptr(work), C.c_int(batch), C.c_int(seq), C.c_int(hidden), C.c_int(heads),
                                        C.c_int(ffn), C.c_float(eps), C.c_int(threads or self.max_threads))
        return out

    def map_unary_f32(self, op, x):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        self.lib.orc_map_unary_f32(C.c_int(op), _ptr(x), _ptr(y), C.c_long(x.size))
        return y

    def map_binary_f32(self, op, a, b):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        y = np.empty_like(a)
        self.lib.orc_map_binary_f32(C.c_int(op), _ptr(a), _ptr(b), _ptr(y), C.c_long(a.size))
        return y

    def map_binary_i32(self, op, a, b):
        a = np.ascontiguousarray(a, np.int32)
        b = np.ascontiguousarray(b, np.int32)
        y = np.empty_like(a)
        self.lib.orc_map_binary_i32(C.c_int(op), _ptr(a), _ptr(b), _ptr(y), C.c_long(a.size))
        return y
