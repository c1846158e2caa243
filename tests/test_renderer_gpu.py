"""Generated kernels on the GPU: render -> compile -> RuntimeFactory -> Program::execute, the
three boundary hooks of tensor/src/realize.rs:1056-1059, compared with the CPU oracle on the
same seeded inputs.  Tolerances from the north star: bit-exact for integer/index ops,
<= 1e-5 relative for f32 elementwise, <= 1e-4 relative for f32 reductions, <= 2e-2 for bf16
GEMM with fp32 accumulate."""
import numpy as np
import pytest

import morok_amd
from morok_amd import synth, uop as U
from tests import kernels_lib as KL

pytestmark = pytest.mark.gpu

UNARY_IDS = {"neg": 0, "abs": 1, "sqrt": 2, "rsqrt": 3, "reciprocal": 4, "exp": 5, "exp2": 6, "log": 7, "log2": 8,
             "sin": 9, "cos": 10, "tan": 11, "floor": 12, "ceil": 13, "trunc": 14, "round": 15, "erf": 16, "sign": 17,
             "square": 18}
BINARY_F_IDS = {"add": 0, "sub": 1, "mul": 2, "fdiv": 3, "mod": 4, "max": 5, "pow": 6}
BINARY_I_IDS = {"add": 0, "sub": 1, "mul": 2, "idiv": 3, "mod": 4, "max": 5, "and": 7, "or": 8, "xor": 9, "shl": 10,
                "shr": 11}


def run(dev, kernel, name, out_shape, out_dtype, inputs, vals=()):
    spec = U.render(kernel, name, dev.device_id)
    prog = morok_amd.Program.create(morok_amd.compile_spec(spec), dev.device_id)
    out = dev.buffer(int(np.prod(out_shape)) * np.dtype(out_dtype).itemsize)
    bufs = [out] + [morok_amd.Buffer.from_numpy(a, dev.device_id) for a in inputs]
    prog.execute(bufs, vals)  # launch sizes recorded by the renderer
    return out.copyout(out_dtype, out_shape)


def rel_err(y, ref):
    return np.abs(y - ref) / np.maximum(np.abs(ref), 1e-30)


@pytest.mark.parametrize("op", sorted(UNARY_IDS))
def test_unary_f32_parity(dev, oracle, op):
    n = 5000  # not a multiple of the block: exercises the gated tail
    if op in ("sqrt", "rsqrt", "log", "log2"):
        x = synth.uniform((n,), 21, 0, 0.01, 50.0)
    elif op == "reciprocal":
        x = synth.uniform((n,), 21, 0, 0.5, 50.0) * np.where(synth.uniform((n,), 21, 9) > 0, 1, -1).astype(np.float32)
    elif op in ("exp", "exp2"):
        x = synth.uniform((n,), 21, 0, -20.0, 20.0)
    elif op == "tan":
        x = synth.uniform((n,), 21, 0, -1.4, 1.4)
    else:
        x = synth.uniform((n,), 21, 0, -30.0, 30.0)
    y = run(dev, KL.elementwise_unary(op, n), "u_" + op, (n,), np.float32, [x])
    ref = oracle.map_unary_f32(UNARY_IDS[op], x)
    if op in ("neg", "abs", "floor", "ceil", "trunc", "round", "sign", "square", "sqrt"):
        assert np.array_equal(y, ref)  # exactly rounded or exact operations
    elif op in ("sin", "cos"):
        assert np.abs(y - ref).max() <= 1e-5  # absolute near the zeros of the function
    else:
        assert rel_err(y, ref).max() <= 1e-5, rel_err(y, ref).max()


@pytest.mark.parametrize("op", sorted(BINARY_F_IDS))
def test_binary_f32_parity(dev, oracle, op):
    n = 4099
    a = synth.uniform((n,), 22, 0, -8.0, 8.0)
    b = synth.uniform((n,), 22, 1, 0.25, 4.0)
    if op == "pow":
        a = np.abs(a) + np.float32(0.1)
    y = run(dev, KL.elementwise_binary(op, n), "b_" + op, (n,), np.float32, [a, b])
    ref = oracle.map_binary_f32(BINARY_F_IDS[op], a, b)
    if op in ("add", "sub", "mul", "fdiv", "max", "mod"):
        assert np.array_equal(y, ref)  # IEEE-exact operations
    else:
        assert rel_err(y, ref).max() <= 1e-5


@pytest.mark.parametrize("op", sorted(BINARY_I_IDS))
def test_binary_i32_bit_exact(dev, oracle, op):
    n = 3001
    a = synth.randint((n,), 23, 0, high=200001) - 100000
    b = synth.randint((n,), 23, 1, high=2001) - 1000
    if op in ("idiv", "mod"):
        b = np.where(b == 0, 7, b).astype(np.int32)  # C truncating semantics for negatives (ir/src/types.rs:625-646)
    if op in ("shl", "shr"):
        b = (np.abs(b) % 12).astype(np.int32)
    if op == "mul":
        a = (a % 20000).astype(np.int32)
    y = run(dev, KL.elementwise_binary(op, n, U.i32, out_dt=U.i32), "bi_" + op, (n,), np.int32, [a, b])
    assert np.array_equal(y, oracle.map_binary_i32(BINARY_I_IDS[op], a, b))


def test_comparison_to_float_cast(dev):
    n = 1000
    a = synth.uniform((n,), 24, 0)
    b = synth.uniform((n,), 24, 1)
    y = run(dev, KL.elementwise_binary("lt", n, U.f32, out_dt=U.f32), "cmp", (n,), np.float32, [a, b])
    assert np.array_equal(y, (a < b).astype(np.float32))


@pytest.mark.parametrize("form", [True, False])
@pytest.mark.parametrize("op", ["max", "add"])
def test_row_reduce_parity(dev, form, op):
    rows, cols = 150, 777
    x = synth.normal((rows, cols), 25, 0, sigma=2.0)
    y = run(dev, KL.row_reduce(op, rows, cols, form), "rr", (rows,), np.float32, [x])
    if op == "max":
        assert np.array_equal(y, x.max(-1))
    else:
        # same left-to-right f32 accumulation as the CPU kernel
        ref = np.zeros(rows, np.float32)
        for c in range(cols):
            ref += x[:, c]
        assert rel_err(y, ref).max() <= 1e-4
        assert np.array_equal(y, ref)


def test_three_kernel_softmax_matches_oracle_and_fused(dev, oracle):
    rows, cols = 96, 1000
    x = synth.normal((rows, cols), 2, 0, sigma=2.0)
    k1, k2, k3 = KL.softmax_kernels(rows, cols)
    m = run(dev, k1, "r_max", (rows,), np.float32, [x])
    s = run(dev, k2, "r_expsum", (rows,), np.float32, [x, m])
    y = run(dev, k3, "E_div", (rows, cols), np.float32, [x, m, s])
    ref = oracle.softmax_f32(x)
    assert np.array_equal(m, x.max(-1))
    big = ref > 1e-30
    assert rel_err(y, ref)[big].max() <= 1e-5


@pytest.mark.parametrize("size,tol", [(128, 0.5), (256, 1.0), (512, 2.0), (1024, 3.0)])
def test_matmul_f32_reference_generators(dev, oracle, size, tol):
    # the reference's validated square cases incl. configs[0]'s 1024 x 1024 shape
    # (tensor/src/test/unit/matmul.rs:24-41,669-677)
    x = np.arange(size * size)
    a = ((x % 31).astype(np.float32) * np.float32(0.05) - np.float32(0.8)).reshape(size, size)
    b = ((x % 37).astype(np.float32) * np.float32(0.04) - np.float32(0.7)).reshape(size, size)
    c = run(dev, KL.matmul_f32_upcast4x4(size, size, size), "r_mm", (size, size), np.float32, [a, b])
    ref = oracle.matmul_f32(a, b)
    assert np.abs(c - a.astype(np.float64) @ b.astype(np.float64)).max() < tol  # the reference's own bound
    assert np.array_equal(c, ref)  # same sequential fmaf chain per element as the CPU kernel


def test_matmul_f32_config0_uniform_inputs(dev, oracle):
    # configs[0]: A[1024x1024] @ B[1024x1024], entries uniform(-1, 1) from seed 1
    a = synth.uniform((1024, 1024), 1, 0)
    b = synth.uniform((1024, 1024), 1, 1)
    c = run(dev, KL.matmul_f32_upcast4x4(1024, 1024, 1024), "r_mm", (1024, 1024), np.float32, [a, b])
    ref = oracle.matmul_f32(a, b)
    assert (np.abs(c - ref) / np.maximum(np.abs(ref), 1e-3)).max() <= 1e-4
    assert np.array_equal(c, ref)


@pytest.mark.parametrize("shape", [(16, 16, 32), (64, 48, 128), (128, 128, 256)])
def test_wmma_gemm_bf16_parity(dev, oracle, shape):
    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 0)
    b = synth.normal_bf16((K, N), 3, 1)
    c = run(dev, KL.wmma_gemm_bf16(M, N, K), "r_wmma", (M, N), np.uint16, [a, b])
    cf, rf = synth.from_bf16(c), synth.from_bf16(oracle.gemm_bf16(a, b))
    assert np.abs(cf - rf).max() <= 2e-2 * np.abs(rf).max()
    assert np.all(np.abs(cf - rf) <= np.abs(rf) * 2**-7 + 1e-3)
    # one-hot operands pin the lane <-> element mapping of the tensor-core operands exactly
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 5) % K] = 1
    c1 = run(dev, KL.wmma_gemm_bf16(M, N, K), "r_wmma", (M, N), np.uint16, [synth.to_bf16(a1), b])
    assert np.array_equal(c1, b[(np.arange(M) * 5) % K])


def test_wave_reduce_row_sum(dev):
    rows, cols = 40, 512
    x = synth.normal((rows, cols), 26, 0)
    y = run(dev, KL.wave_row_sum(rows, cols), "r_wave", (rows,), np.float32, [x])
    ref = x.astype(np.float64).sum(-1)
    assert np.abs(y - ref).max() <= 1e-4 * np.abs(x).sum(-1).max()
    ones = np.ones((rows, cols), np.float32)
    assert np.all(run(dev, KL.wave_row_sum(rows, cols), "r_wave", (rows,), np.float32, [ones]) == cols)


def test_async_copy_and_transposing_load(dev):
    """The documented lane maps of the local-memory extension ops: a direct copy lays lane i's 16
    bytes 16 i bytes into the destination, and within a group of 16 lanes a transposing load hands
    lane i column i of the 4 x 16 block whose row i / 4, columns 4 (i % 4) .. + 3 it addressed."""
    x = (np.arange(512, dtype=np.uint16) * 7 + 3).astype(np.uint16)
    y = run(dev, KL.async_copy_transposing_load(), "tr", (64, 4), np.uint16, [x])
    m = x.reshape(16, 32)
    lanes = np.arange(64)
    want = np.stack([m[4 * (lanes // 16) + e, lanes % 16] for e in range(4)], axis=1)
    assert np.array_equal(y, want)


def test_local_memory_transpose(dev):
    n = 16
    x = synth.normal((n, n), 27, 0)
    y = run(dev, KL.local_memory_transpose(n), "t", (n, n), np.float32, [x])
    assert np.array_equal(y, x.T)


def test_variables_positional_vals(dev):
    k = U.Kernel()
    out = k.param(0, U.f32, 1024)
    n = k.define_var("n", U.i32, 1, 1024)
    off = k.define_var("off", U.i64, 0, 1 << 40)
    l = k.special("lidx0", 256)
    g = k.special("gidx0", 4)
    idx = k.add(k.mul(g, k.const(256)), l)
    k.if_(k.binary("lt", idx, n))
    k.store(k.index(out, idx), k.cast(k.binary("sub", k.add(k.cast(idx, U.i64), off), k.const(1 << 33, U.i64)), U.f32))
    k.endif()
    spec = U.render(k, "v", dev.device_id)
    prog = morok_amd.Program.create(morok_amd.compile_spec(spec), dev.device_id)
    out_b = dev.buffer(4096, zero_init=True)
    prog.execute([out_b], [700, (1 << 33) + 5])  # a value that needs all 64 bits
    y = out_b.copyout(np.float32)
    assert np.array_equal(y[:700], np.arange(700, dtype=np.float32) + 5) and not y[700:].any()


@pytest.mark.parametrize("tc,shape,out", [(3, (64, 160, 128), U.BF16), (3, (16, 16, 32), U.BF16), (5, (48, 32, 64), U.BF16),
                                          (3, (80, 48, 96), U.F32)])
def test_tc_apply_matmul_from_tables(dev, oracle, tc, shape, out):
    """The tensor-core matmul built from the CDNA tables (opts + swizzle) on the GPU."""
    from morok_amd import sched

    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 10)
    b = synth.normal_bf16((K, N), 3, 11)
    kern = sched.build_wmma_matmul(tc, M, N, K, out)
    np_out = np.uint16 if out == U.BF16 else np.float32
    c = run(dev, kern, "r_tc", (M, N), np_out, [a, b])
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    cf = synth.from_bf16(c) if out == U.BF16 else c
    assert np.abs(cf - ref).max() <= 2e-2 * np.abs(ref).max()
    if out == U.F32:
        assert np.abs(cf - ref).max() <= 1e-4 * np.abs(ref).max()
    # one-hot rows pin the operand gather exactly
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    c1 = run(dev, kern, "r_tc", (M, N), np_out, [synth.to_bf16(a1), b])
    want = b[(np.arange(M) * 7) % K]
    assert np.array_equal(c1, want if out == U.BF16 else synth.from_bf16(want))


@pytest.mark.parametrize("tc,shape,out", [(3, (128, 128, 32), U.BF16), (3, (256, 384, 160), U.BF16), (3, (128, 256, 1024), U.F32),
                                          (5, (128, 128, 48), U.BF16), (5, (256, 128, 96), U.BF16)])
def test_tc_matmul_staged_through_local_memory(dev, oracle, tc, shape, out):
    """The generated tensor-core matmul with a 2 x 2-wave workgroup, both operands copied
    through LDS (B with pairs of K rows interleaved, or as plain rows when the K tile is 16
    deep) and two barriers per K step: against float64, the
    register-only generated kernel (same products, same K order: the same bits) and one-hot
    operands that pin the copy and fragment indexing exactly."""
    from morok_amd import sched

    M, N, K = shape
    a = synth.normal_bf16((M, K), 3, 12)
    b = synth.normal_bf16((K, N), 3, 13)
    kern = sched.build_wmma_matmul_lds(tc, M, N, K, out)
    np_out = np.uint16 if out == U.BF16 else np.float32
    c = run(dev, kern, "r_tc_lds", (M, N), np_out, [a, b])
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    cf = synth.from_bf16(c) if out == U.BF16 else c
    assert np.abs(cf - ref).max() <= 2e-2 * np.abs(ref).max()
    plain = run(dev, sched.build_wmma_matmul(tc, M, N, K, out), "r_tc", (M, N), np_out, [a, b])
    assert np.array_equal(c, plain)
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    c1 = run(dev, kern, "r_tc_lds", (M, N), np_out, [synth.to_bf16(a1), b])
    want = b[(np.arange(M) * 7) % K]
    assert np.array_equal(c1, want if out == U.BF16 else synth.from_bf16(want))


@pytest.mark.parametrize("opts", [(1, 1, 1, 1, 0), (1, 1, 2, 4, 1), (1, 4, 4, 1, 2), (4, 1, 1, 4, 0), (2, 4, 2, 2, 2),
                                  (4, 2, 2, 4, 2), (2, 2, 8, 4, 0), (2, 1, 2, 8, 2), (4, 4, 2, 2, 0), (1, 2, 4, 2, 1), (2, 2, 2, 2, 4)])
def test_tc_matmul_lds_choices_agree(dev, opts):
    """Every LOCAL / UPCAST / UNROLL choice of the LDS-staged tensor-core kernel computes the same
    products in the same K order: the bits of the register-only generated kernel, and one-hot
    operands come back exactly (copy and fragment indexing of each variant)."""
    from morok_amd import sched

    M, N, K = 512, 256, 256
    a = synth.normal_bf16((M, K), 5, 21)
    b = synth.normal_bf16((K, N), 5, 22)
    kern = sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts)
    c = run(dev, kern, "r_tc_lds", (M, N), np.uint16, [a, b])
    plain = run(dev, sched.build_wmma_matmul(3, M, N, K, U.BF16), "r_tc", (M, N), np.uint16, [a, b])
    assert np.array_equal(c, plain)
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    c1 = run(dev, kern, "r_tc_lds", (M, N), np.uint16, [synth.to_bf16(a1), b])
    assert np.array_equal(c1, b[(np.arange(M) * 7) % K])


@pytest.mark.parametrize("tc,kind,one", [(0, 1, 0x3C), (1, 0, 0x38)])
@pytest.mark.parametrize("shape", [(16, 16, 32), (64, 80, 128), (48, 32, 256)])
def test_tc_apply_matmul_fp8(dev, oracle, tc, kind, one, shape):
    """The two 8-bit-float tensor cores of the CDNA4 table (E5M2 first, then E4M3): operands are
    byte codes, eight per lane, the accumulator is f32.  Products of 8-bit floats are exact in f32
    and the oracle adds them one by one.  The matrix core adds the 32 products of a K step as one
    block, aligned to the block's largest product, and drops what lies more than about 11.6 bits
    below it (measured: error <= 2^-11.6 of the largest product per block over the formats' whole
    range, none at all when the operands span a few binades).  So: operands within [0.5, 2) give
    the float64 result exactly; operands over the wide range stay within 2^-11 of the largest
    product per block of 32, summed over the blocks; one-hot rows of 1.0 return the decoded rows
    of B exactly."""
    from morok_amd import sched

    M, N, K = shape
    rng = np.random.default_rng(97 + kind)
    kern = sched.build_wmma_matmul(tc, M, N, K, U.F32)

    def codes(lo, hi, shp):
        return rng.integers(lo, hi, shp).astype(np.uint8) | (rng.integers(0, 2, shp).astype(np.uint8) << 7)

    one_code, two_code = one, one + (8 if kind == 0 else 4)              # 1.0 and 2.0
    a, b = codes(one_code - (two_code - one_code), two_code, (M, K)), codes(one_code - (two_code - one_code), two_code, (K, N))
    c = run(dev, kern, "r_tc8", (M, N), np.float32, [a, b])
    af, bf = oracle.fp8_to_f32(kind, a).astype(np.float64), oracle.fp8_to_f32(kind, b).astype(np.float64)
    assert np.abs(af).min() >= 0.5 and np.abs(af).max() < 2.0
    assert np.array_equal(c, (af @ bf).astype(np.float32)) and np.array_equal(c, oracle.matmul_fp8_f32(kind, a, b))
    a, b = codes(0x08, 0x60, (M, K)), codes(0x08, 0x60, (K, N))
    c = run(dev, kern, "r_tc8", (M, N), np.float32, [a, b])
    ref = oracle.matmul_fp8_f32(kind, a, b)
    af, bf = oracle.fp8_to_f32(kind, a).astype(np.float64), oracle.fp8_to_f32(kind, b).astype(np.float64)
    terms = np.abs(af[:, :, None] * bf[None, :, :]).reshape(M, K // 32, 32, N)
    bound = 2.0 ** -11 * terms.max(2).sum(1) + 1e-6 * np.abs(af) @ np.abs(bf)
    assert np.all(np.abs(c - ref) <= bound)
    a1 = np.zeros((M, K), np.uint8)
    a1[np.arange(M), (np.arange(M) * 5) % K] = one
    c1 = run(dev, kern, "r_tc8", (M, N), np.float32, [a1, b])
    assert np.array_equal(c1, oracle.fp8_to_f32(kind, b)[(np.arange(M) * 5) % K])


@pytest.mark.parametrize("shape,opts", [((512, 512, 256), (2, 2, 2, 2, 0, 2)), ((256, 384, 64), (2, 2, 4, 4, 0, 2)),
                                        ((128, 192, 128), (1, 4, 4, 1, 0, 2)), ((512, 512, 192), (4, 4, 4, 4, 0, 2)),
                                        ((512, 256, 320), (2, 2, 8, 8, 0, 2)), ((256, 512, 256), (2, 4, 8, 4, 0, 2)),
                                        ((192, 128, 448), (1, 1, 4, 4, 0, 2)), ((768, 256, 128), (2, 2, 8, 4, 2, 2)),
                                        ((256, 1024, 128), (4, 2, 4, 8, 0, 2)), ((1536, 768, 64), (2, 2, 8, 8, 0, 2)),
                                        # a third stage of the second operand's tile (copies spread over the whole step)
                                        ((512, 256, 320), (2, 2, 8, 8, 0, 3)), ((256, 512, 192), (2, 2, 8, 8, 0, 3)), ((256, 256, 256), (1, 4, 8, 2, 0, 3)),
                                        ((384, 128, 448), (1, 1, 4, 4, 0, 3)), ((768, 512, 1024), (2, 2, 8, 4, 0, 3))])
def test_tc_matmul_direct_copy_choices_agree(dev, shape, opts):
    """The variant whose tiles arrive by direct global -> local copies (two stages, transposing B
    reads, operands swapped at the tensor core, tiles assigned per XCD) computes the same products
    in the same K order as the register-only generated kernel: same bits, one-hot operands come
    back exactly, and nothing outside the operands is read or outside the result written (NaN
    patterns behind each of them would surface).  K steps of 1, 2, 3 and more cover the prologue,
    the last copy and the steady state; tile counts that 8 and 4 do not divide cover the mapping."""
    from morok_amd import sched

    M, N, K = shape
    a = synth.normal_bf16((M, K), 9, 41)
    b = synth.normal_bf16((K, N), 9, 42)
    kern = sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts)
    nan = np.uint16(0x7FC0)

    def fenced(x):
        big = np.full(x.size + 4096, nan, np.uint16)
        big[:x.size] = x.ravel()
        return morok_amd.Buffer.from_numpy(big)

    def run_fenced(av):
        bc = morok_amd.Buffer.from_numpy(np.full(M * N + 4096, nan, np.uint16))
        k = morok_amd.Kernel.get_or_compile(kern, "r_tc_dma")
        plan = morok_amd.ExecutionPlan()
        plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(fenced(av)), plan.add_buffer(fenced(b))])
        plan.build().execute()
        got = bc.copyout(np.uint16, (M * N + 4096,))
        assert np.all(got[M * N:] == nan)
        return got[:M * N].reshape(M, N)

    plain = run(dev, sched.build_wmma_matmul(3, M, N, K, U.BF16), "r_tc", (M, N), np.uint16, [a, b])
    assert np.array_equal(run_fenced(a), plain)
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    assert np.array_equal(run_fenced(synth.to_bf16(a1)), b[(np.arange(M) * 7) % K])


@pytest.mark.parametrize("shape,opts", [((512, 512, 256), (2, 4, 4, 2, 0, 2)), ((256, 256, 64), (2, 2, 2, 2, 0, 2)), ((512, 256, 192), (4, 2, 2, 4, 0, 2)),
                                        ((256, 512, 128), (1, 4, 2, 1, 0, 2)), ((768, 384, 320), (2, 2, 4, 2, 0, 2))])
def test_tc_matmul_32x32x16_tiles(dev, shape, opts):
    """The 32x32x16 tensor-core entries (gfx950 additions behind the reference's table): the
    register-only kernel and the direct-copy variant built from them agree bit for bit with each
    other, with the 16x16x32 kernels (the matrix core adds the 16-deep and the 32-deep blocks of
    products in the same order) and with the hand-written GEMM, which uses the same instruction."""
    from morok_amd import ops, sched

    M, N, K = shape
    a, b = synth.normal_bf16((M, K), 9, 61), synth.normal_bf16((K, N), 9, 62)
    plain32 = run(dev, sched.build_wmma_matmul(7, M, N, K, U.BF16), "r_tc32", (M, N), np.uint16, [a, b])
    plain16 = run(dev, sched.build_wmma_matmul(3, M, N, K, U.BF16), "r_tc16", (M, N), np.uint16, [a, b])
    dma32 = run(dev, sched.build_wmma_matmul_lds_opts(7, M, N, K, U.BF16, opts), "r_tc32_dma", (M, N), np.uint16, [a, b])
    ba, bb, bc = (morok_amd.Buffer.from_numpy(a), morok_amd.Buffer.from_numpy(b), dev.buffer(M * N * 2))
    ops.gemm_bf16(ba, bb, bc, M, N, K, dev.device_id)
    hand = bc.copyout(np.uint16, (M, N))
    assert np.array_equal(plain32, plain16) and np.array_equal(dma32, plain32) and np.array_equal(hand, plain32)
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    one_hot = run(dev, sched.build_wmma_matmul_lds_opts(7, M, N, K, U.BF16, opts), "r_tc32_dma", (M, N), np.uint16, [synth.to_bf16(a1), b])
    assert np.array_equal(one_hot, b[(np.arange(M) * 7) % K])


def test_tc_matmul_direct_copy_f32_result(dev):
    """An f32 result leaves the accumulators directly (no staging through local memory): the bits
    of the register-only generated kernel with the same result type; f16 operands take the f16
    transposing load."""
    from morok_amd import sched

    M, N, K = 256, 256, 192
    a, b = synth.normal_bf16((M, K), 9, 51), synth.normal_bf16((K, N), 9, 52)
    got = run(dev, sched.build_wmma_matmul_lds_opts(3, M, N, K, U.F32, (2, 2, 4, 4, 0, 2)), "r_tc_dma_f32", (M, N), np.float32, [a, b])
    want = run(dev, sched.build_wmma_matmul(3, M, N, K, U.F32), "r_tc", (M, N), np.float32, [a, b])
    assert np.array_equal(got, want)
    ah, bh = synth.normal((M, K), 9, 53).astype(np.float16), synth.normal((K, N), 9, 54).astype(np.float16)
    got = run(dev, sched.build_wmma_matmul_lds_opts(2, M, N, K, U.F16, (2, 4, 4, 2, 0, 2)), "r_tc_dma_h", (M, N), np.float16, [ah, bh])
    want = run(dev, sched.build_wmma_matmul(2, M, N, K, U.F16), "r_tc_h", (M, N), np.float16, [ah, bh])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,opts", [((200, 136, 72), (2, 2, 4, 4, 0)), ((1, 8, 8), (1, 1, 1, 1, 0)), ((130, 264, 200), (2, 2, 2, 2, 2)),
                                        ((257, 256, 64), (4, 4, 4, 4, 0)), ((128, 128, 40), (2, 2, 4, 4, 0)), ((100, 128, 64), (1, 4, 4, 1, 2))])
def test_tc_matmul_lds_padded_shapes(dev, shape, opts):
    """PADTO: extents the workgroup tile does not divide.  Loads past the operands are gated
    to zero and stores past the result skipped: values against float64, one-hot rows exact,
    and memory behind the result and the operands untouched / unread (NaN patterns placed
    there would surface in the result)."""
    from morok_amd import sched

    M, N, K = shape
    a = synth.normal_bf16((M, K), 6, 31)
    b = synth.normal_bf16((K, N), 6, 32)
    kern = sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts)
    # operands and result each sit in the front of a larger NaN-filled buffer
    nan = np.uint16(0x7FC0)
    abig = np.full(M * K + 4096, nan, np.uint16); abig[:M * K] = a.ravel()
    bbig = np.full(K * N + 4096, nan, np.uint16); bbig[:K * N] = b.ravel()
    ba, bb = morok_amd.Buffer.from_numpy(abig), morok_amd.Buffer.from_numpy(bbig)
    bc = morok_amd.Buffer.from_numpy(np.full(M * N + 4096, nan, np.uint16))
    k = morok_amd.Kernel.get_or_compile(kern, "r_tc_pad")
    plan = morok_amd.ExecutionPlan()
    plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(ba), plan.add_buffer(bb)])
    plan.build().execute()
    got = bc.copyout(np.uint16, (M * N + 4096,))
    assert np.all(got[M * N:] == nan)
    c = synth.from_bf16(got[:M * N].reshape(M, N))
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    assert np.all(np.isfinite(c)) and np.abs(c - ref).max() <= 2e-2 * np.abs(ref).max()
    a1 = np.zeros((M, K), np.float32)
    a1[np.arange(M), (np.arange(M) * 7) % K] = 1
    c1 = run(dev, kern, "r_tc_pad", (M, N), np.uint16, [synth.to_bf16(a1), b])
    assert np.array_equal(c1, b[(np.arange(M) * 7) % K])


def test_scheduled_matmul_f32_kernel(dev, oracle):
    from morok_amd import sched

    a = synth.uniform((128, 96), 1, 5)
    b = synth.uniform((96, 192), 1, 6)
    c = run(dev, sched.build_matmul_f32(128, 192, 96), "r_mm", (128, 192), np.float32, [a, b])
    assert np.array_equal(c, oracle.matmul_f32(a, b))


@pytest.mark.parametrize("opts", [[16, 16, 4, 4, 1, 16], [32, 16, 4, 8, 1, 16], [8, 16, 4, 4, 1, 16], [16, 16, 8, 8, 1, 8],
                                  [16, 8, 4, 8, 1, 32]])
def test_matmul_f32_staged_through_local_memory(dev, oracle, opts):
    """GROUP: the workgroup stages A (transposed) and B tiles through local memory; every tile
    choice computes the same sums in the same k order as the kernel that reads global memory
    directly (bit-identical to it) and matches the CPU oracle within the f32 reduction tolerance."""
    from morok_amd import sched

    M, N, K = 256, 384, 160
    a, b = synth.uniform((M, K), 55, 0), synth.uniform((K, N), 55, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a, dev.device_id), morok_amd.Buffer.from_numpy(b, dev.device_id)

    def run_opts(o):
        out = dev.buffer(M * N * 4 + 4096)
        out.copyin(np.full(M * N + 1024, np.nan, np.float32))
        k = morok_amd.Kernel.get_or_compile(sched.build_matmul_f32_opts(M, N, K, o), "mm_" + "_".join(map(str, o)))
        plan = morok_amd.ExecutionPlan()
        plan.add_kernel(k, [plan.add_buffer(out), plan.add_buffer(ba), plan.add_buffer(bb)])
        plan.build().execute()
        raw = out.copyout(np.float32)
        assert np.all(np.isnan(raw[M * N:]))   # nothing written behind the result
        return raw[: M * N].reshape(M, N)

    got = run_opts(opts)
    assert np.array_equal(got, run_opts([16, 16, 4, 4, 1, 0]))
    ref = oracle.matmul_f32(a, b)
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
