"""Direct entry points of the hand-written kernels (device buffers in, device buffers out)."""
import ctypes as C

from ._ffi import check, lib
from .device import Buffer


def _p(b):
    return C.c_void_p(b.ptr if isinstance(b, Buffer) else int(b))


def _need(b, nbytes, what):
    """Host-side shape check before a hand-written kernel is launched: a Buffer that is too
    small for the stated shape is refused here instead of faulting on the GPU.  Raw device
    addresses carry no size and are taken on trust."""
    if isinstance(b, Buffer) and b.size < nbytes:
        raise ValueError(f"{what}: buffer of {b.size} bytes is smaller than the {nbytes} bytes the shape needs")


def softmax_f32(x, y, rows, cols, device_id=0, variant=0):
    """Fused row softmax (Tensor::softmax, tensor/src/activation.rs:90-101), last axis."""
    for b, w in ((x, "softmax input"), (y, "softmax output")):
        _need(b, rows * cols * 4, w)
    check(lib.mrk_hip_softmax_f32_variant(device_id, _p(x), _p(y), rows, cols, variant))


def gemm_bf16(a, b, c, m, n, k, device_id=0, variant=0):
    """c[m,n] = a[m,k] @ b[k,n], bf16 row-major, f32 accumulate (Tensor::matmul on bf16,
    tensor/src/matmul.rs:82-110)."""
    _need(a, m * k * 2, "gemm A")
    _need(b, k * n * 2, "gemm B")
    _need(c, m * n * 2, "gemm C")
    check(lib.mrk_hip_gemm_bf16_variant(device_id, _p(a), _p(b), _p(c), m, n, k, variant))


def gemm_bf16_nt(a, bt, c, m, n, k, device_id=0):
    """c[m,n] = a[m,k] @ bt[n,k]^T: the second operand as a Linear layer stores its weight
    ([out_features, in_features], k contiguous).  The same bits as gemm_bf16 on the transposed
    matrix; tiled kernels only (n and k multiples of 8, no split-K shapes)."""
    _need(a, m * k * 2, "gemm_bf16_nt a")
    _need(bt, n * k * 2, "gemm_bf16_nt bt")
    _need(c, m * n * 2, "gemm_bf16_nt c")
    check(lib.mrk_hip_gemm_bf16_nt(device_id, _p(a), _p(bt), _p(c), m, n, k))


def gemm_f16(a, b, c, m, n, k, device_id=0):
    """c[m,n] = a[m,k] @ b[k,n] on IEEE half precision operands, f32 accumulate, f16 result: the
    hand-written tiled kernels around v_mfma_f32_16x16x32_f16 (Tensor::matmul on f16)."""
    _need(a, m * k * 2, "gemm A")
    _need(b, k * n * 2, "gemm B")
    _need(c, m * n * 2, "gemm C")
    check(lib.mrk_hip_gemm_f16(device_id, _p(a), _p(b), _p(c), m, n, k))


def gemm_f16_nt(a, bt, c, m, n, k, device_id=0):
    """c[m,n] = a[m,k] @ bt[n,k]^T on f16 operands (second operand as a Linear layer stores it)."""
    _need(a, m * k * 2, "gemm_f16_nt a")
    _need(bt, n * k * 2, "gemm_f16_nt bt")
    _need(c, m * n * 2, "gemm_f16_nt c")
    check(lib.mrk_hip_gemm_f16_nt(device_id, _p(a), _p(bt), _p(c), m, n, k))


def gemm_bf16_noalloc(a, b, c, m, n, k, device_id=0):
    """gemm_bf16 without any device allocation: split-K partials go to the library's fixed
    device scratch (for callers under graph capture or in loops that must not allocate)."""
    _need(a, m * k * 2, "gemm A")
    _need(b, k * n * 2, "gemm B")
    _need(c, m * n * 2, "gemm C")
    check(lib.mrk_hip_gemm_bf16_noalloc(device_id, _p(a), _p(b), _p(c), m, n, k))


def gemm_bf16_swiglu(a, w, c, m, f, k, device_id=0):
    """c[m,f] = silu(a @ w[:, :f]) * (a @ w[:, f:]) for w [k, 2f] = gate | up, the gate applied in the
    product kernel's epilogue."""
    _need(a, m * k * 2, "gemm A")
    _need(w, k * 2 * f * 2, "gemm W (gate | up)")
    _need(c, m * f * 2, "gemm C")
    check(lib.mrk_hip_gemm_bf16_swiglu(device_id, _p(a), _p(w), _p(c), m, f, k))


def linear_bf16(x, w, bias, y, m, n, k, device_id=0):
    """y[m, n] = x[m, k] @ w[n, k].T + bias[n] with the weight and bias as a Linear layer stores them; bias may be
    None.  The bias is added in the product kernel's epilogue (the bits of the product followed by the add)."""
    _need(x, m * k * 2, "linear_bf16 x")
    _need(w, n * k * 2, "linear_bf16 w")
    _need(y, m * n * 2, "linear_bf16 y")
    if bias is not None:
        _need(bias, n * 2, "linear_bf16 bias")
    check(lib.mrk_hip_linear_bf16(device_id, _p(x), _p(w), _p(bias) if bias is not None else None, _p(y), m, n, k))


def gemm_bf16_residual(a, b, r, c, m, n, k, device_id=0):
    """c[m,n] = a[m,k] @ b[k,n] + r[m,n]: the residual added in the product kernel's epilogue,
    same bits as gemm_bf16 followed by an elementwise add."""
    _need(a, m * k * 2, "gemm A")
    _need(b, k * n * 2, "gemm B")
    _need(r, m * n * 2, "gemm R")
    _need(c, m * n * 2, "gemm C")
    check(lib.mrk_hip_gemm_bf16_residual(device_id, _p(a), _p(b), _p(r), _p(c), m, n, k))


def gemm_bf16_rope(a, b, cos, sin, c_rot, c_rest, m, n, k, split, seq, device_id=0):
    """c_rot[m, split] = rotary embedding (heads of 128 columns, non-interleaved, position = row % seq,
    cos / sin [seq, 64] f32) of the first `split` columns of a[m,k] @ b[k,n]; c_rest[m, n - split] =
    the remaining columns, unrotated.  One kernel: the rotation runs in the product's epilogue."""
    _need(a, m * k * 2, "gemm A")
    _need(b, k * n * 2, "gemm B")
    _need(cos, seq * 64 * 4, "rope cos")
    _need(sin, seq * 64 * 4, "rope sin")
    _need(c_rot, m * split * 2, "gemm C (rotated part)")
    if split < n:
        _need(c_rest, m * (n - split) * 2, "gemm C (rest)")
    check(lib.mrk_hip_gemm_bf16_rope(device_id, _p(a), _p(b), _p(cos), _p(sin), _p(c_rot), _p(c_rest) if split < n else None, m, n, k,
                                     split, seq))


def flash_attn_fwd_bf16(q, k, v, o, batch, heads, sq, sk, d, scale, causal=True, device_id=0):
    """Fused SDPA forward (Tensor::scaled_dot_product_attention, tensor/src/transformer.rs:78-137)."""
    _need(q, batch * heads * sq * d * 2, "attention Q")
    _need(o, batch * heads * sq * d * 2, "attention O")
    _need(k, batch * heads * sk * d * 2, "attention K")
    _need(v, batch * heads * sk * d * 2, "attention V")
    check(lib.mrk_hip_flash_attn_fwd_bf16(device_id, _p(q), _p(k), _p(v), _p(o), batch, heads, sq, sk, d, scale,
                                          int(causal)))


def flash_attn_fwd_bf16_strided(q, k, v, o, batch, heads, sq, sk, d, scale, strides, offsets=(0, 0, 0, 0), causal=True,
                                device_id=0):
    """The fused SDPA forward over views: `strides` = (batch, head, row) element strides of q, k,
    v, o (12 values), `offsets` = element offset of each operand's first element inside its
    buffer.  Each Buffer must hold the last element its view reaches."""
    strides = [int(x) for x in strides]
    if len(strides) != 12 or len(offsets) != 4:
        raise ValueError("flash_attn_fwd_bf16_strided takes 12 strides and 4 offsets")
    ptrs = []
    for i, (b, rows, what) in enumerate(((q, sq, "attention Q"), (k, sk, "attention K"), (v, sk, "attention V"),
                                         (o, sq, "attention O"))):
        sb, sh, sr = strides[3 * i:3 * i + 3]
        off = int(offsets[i])
        if off < 0 or off % 8:
            raise ValueError(f"{what}: offset {off} must be a non-negative multiple of 8 elements")
        if batch and heads and rows:
            _need(b, (off + (batch - 1) * sb + (heads - 1) * sh + (rows - 1) * sr + d) * 2, what)
        ptrs.append(C.c_void_p((b.ptr if isinstance(b, Buffer) else int(b)) + off * 2))
    arr = (C.c_int64 * 12)(*strides)
    check(lib.mrk_hip_flash_attn_fwd_bf16_strided(device_id, ptrs[0], ptrs[1], ptrs[2], ptrs[3], batch, heads, sq, sk, d,
                                                  scale, int(causal), arr))


def flash_attn_fwd_bf16_ex(q, k, v, o, batch, heads, sq, sk, d, scale, causal=False, mask=None, mask_kind=0,
                           mask_strides=(0, 0, 0), softcap=0.0, strides=None, device_id=0):
    """The fused SDPA forward with attn_mask and / or softcap inside the kernel
    (tensor/src/transformer.rs:112-132).  mask_kind 1: Bool bytes (nonzero = attend), 2: additive
    bf16; mask_strides = element strides of the mask per batch, head and query row (0 broadcasts),
    keys contiguous.  `strides`: as flash_attn_fwd_bf16_strided, or None for dense operands."""
    if strides is None:
        _need(q, batch * heads * sq * d * 2, "attention Q")
        _need(o, batch * heads * sq * d * 2, "attention O")
        _need(k, batch * heads * sk * d * 2, "attention K")
        _need(v, batch * heads * sk * d * 2, "attention V")
        arr = None
    else:
        strides = [int(x) for x in strides]
        if len(strides) != 12:
            raise ValueError("flash_attn_fwd_bf16_ex takes 12 strides")
        for i, (b, rows, what) in enumerate(((q, sq, "attention Q"), (k, sk, "attention K"), (v, sk, "attention V"),
                                             (o, sq, "attention O"))):
            sb, sh, sr = strides[3 * i:3 * i + 3]
            if batch and heads and rows:
                _need(b, ((batch - 1) * sb + (heads - 1) * sh + (rows - 1) * sr + d) * 2, what)
        arr = (C.c_int64 * 12)(*strides)
    marr = None
    if mask_kind:
        if mask is None or len(mask_strides) != 3:
            raise ValueError("flash_attn_fwd_bf16_ex: a mask kind needs a mask and 3 mask strides")
        mb, mh, mr = (int(x) for x in mask_strides)
        if batch and heads and sq:
            _need(mask, ((batch - 1) * mb + (heads - 1) * mh + (sq - 1) * mr + sk) * (2 if mask_kind == 2 else 1), "attention mask")
        marr = (C.c_int64 * 3)(mb, mh, mr)
    check(lib.mrk_hip_flash_attn_fwd_bf16_ex(device_id, _p(q), _p(k), _p(v), _p(o), batch, heads, sq, sk, d, scale, int(causal),
                                             arr, _p(mask) if mask_kind else None, int(mask_kind), marr, float(softcap)))


def fill_normal(buf, n, sigma=1.0, seed=0, tensor_id=0, bf16=False, device_id=0):
    """Device-side synthetic normal(0, sigma) values (benchmark inputs)."""
    _need(buf, n * (2 if bf16 else 4), "fill")
    check(lib.mrk_hip_fill(device_id, _p(buf), n, int(bf16), 1, seed, tensor_id, sigma, 0.0))


def fill_uniform(buf, n, lo=-1.0, hi=1.0, seed=0, tensor_id=0, bf16=False, device_id=0):
    _need(buf, n * (2 if bf16 else 4), "fill")
    check(lib.mrk_hip_fill(device_id, _p(buf), n, int(bf16), 0, seed, tensor_id, lo, hi))


def fill_randint(buf, n, high, seed=0, tensor_id=0, device_id=0):
    _need(buf, n * 4, "fill_randint")
    check(lib.mrk_hip_fill_randint(device_id, _p(buf), n, seed, tensor_id, high))


def copy_kernel(src, dst, nbytes, device_id=0):
    """Streaming copy kernel of known traffic (counter calibration)."""
    _need(src, nbytes, "copy source")
    _need(dst, nbytes, "copy destination")
    check(lib.mrk_hip_copy_kernel(device_id, _p(src), _p(dst), nbytes))


def mfma_ceiling(scratch, workgroups, k_steps, device_id=0, random_operands=True):
    """MFMA-only calibration kernel: the matrix-instruction stream of `workgroups` 256x256 GEMM
    tiles of depth 64 * k_steps, from registers (2 * 256 * 256 * 64 * k_steps flops each)."""
    _need(scratch, 4, "mfma_ceiling scratch")
    check(lib.mrk_hip_mfma_ceiling(device_id, _p(scratch), workgroups, k_steps, 2 if random_operands == "f16" else int(random_operands)))
