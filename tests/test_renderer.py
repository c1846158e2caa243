"""Renderer tests that need no GPU: text assertions in the style of the reference's
renderer tests (codegen/src/test/unit/c.rs:9-278) and compilation of every rendered kernel
for gfx950 with the in-process compiler."""
import pytest

import morok_amd
from morok_amd import MorokHipError, uop as U
from tests import kernels_lib as KL


def _compiles(spec):
    c = morok_amd.compile_spec(spec)
    assert c.src is None and len(c.bytes) > 1000
    return c


def test_elementwise_signature_and_launch_dims():
    spec = U.render(KL.elementwise_unary("exp", 1000), "E_exp")
    src = spec.src
    assert 'extern "C" __global__ void __launch_bounds__(256) E_exp(float* __restrict__ data0, const float* __restrict__ data1)' in src
    assert "blockIdx.x" in src and "threadIdx.x" in src
    assert "expf(" in src
    assert spec.global_size == [4, 1, 1] and spec.local_size == [256, 1, 1]
    assert spec.buf_count == 2 and spec.globals == [0, 1] and spec.outs == [0] and spec.ins == [1]
    assert spec.var_names == []
    _compiles(spec)


def test_default_name_and_bad_name():
    assert U.render(KL.elementwise_unary("neg", 64)).name == "kernel"  # device.rs:192-193
    with pytest.raises(MorokHipError) as e:
        U.render(KL.elementwise_unary("neg", 64), "bad name")
    assert e.value.code == 9


@pytest.mark.parametrize("op,text", [("sqrt", "sqrtf("), ("rsqrt", "(1.0f / sqrtf("), ("reciprocal", "(1.0f / "),
                                     ("exp2", "exp2f("), ("log", "logf("), ("sin", "sinf("), ("round", "rintf("),
                                     ("erf", "erff("), ("abs", "fabsf("), ("trunc", "truncf(")])
def test_unary_op_semantics_text(op, text):
    # codegen/src/c/ops.rs:533-584
    spec = U.render(KL.elementwise_unary(op, 256), "u")
    assert text in spec.src
    _compiles(spec)


def test_binary_op_semantics_text():
    # codegen/src/c/ops.rs:489-531
    assert "fmaxf(" in U.render(KL.elementwise_binary("max", 256), "b").src
    assert "fmodf(" in U.render(KL.elementwise_binary("mod", 256), "b").src
    assert "powf(" in U.render(KL.elementwise_binary("pow", 256), "b").src
    s = U.render(KL.elementwise_binary("max", 256, U.i32), "b").src
    assert "fmaxf" not in s and " > " in s and "?" in s
    s = U.render(KL.elementwise_binary("mod", 256, U.i32), "b").src
    assert "%" in s
    for op in ("add", "idiv", "and", "xor", "shl", "lt"):
        _compiles(U.render(KL.elementwise_binary(op, 256, U.i32, out_dt=U.i32), "b"))


def test_reduce_forms():
    a = U.render(KL.row_reduce("max", 100, 64, use_reduce_node=True), "r_max")
    assert "= -__builtin_inff();" in a.src and "fmaxf(acc" in a.src and "for (int ridx0 = 0; ridx0 < 64; ridx0++) {" in a.src
    b = U.render(KL.row_reduce("add", 100, 64, use_reduce_node=False), "r_sum")
    assert "float reg0[1];" in b.src and "for (int ridx0" in b.src
    _compiles(a)
    _compiles(b)


def test_gated_load_and_store_if():
    src = U.render(KL.elementwise_unary("neg", 1000), "g").src
    assert " ? *(" in src and ": 0.0f)" in src  # gated load with zero alt (ops.rs:186-215)
    assert "if (" in src  # gated store lowered to IF/STORE/ENDIF by line_rewrite_cleanups


def test_local_memory_and_barrier():
    spec = U.render(KL.local_memory_transpose(16), "t")
    assert "__shared__ float local0[256];" in spec.src and "__syncthreads();" in spec.src
    assert spec.local_size == [16, 16, 1]
    _compiles(spec)


def test_vector_ops_and_mulacc():
    spec = U.render(KL.matmul_f32_upcast4x4(128, 128, 64), "mm")
    assert "typedef float mrk_float4 __attribute__((aligned(16), ext_vector_type(4)));" in spec.src
    assert "fmaf(" in spec.src and "*((mrk_float4*)(" in spec.src and "(mrk_float4){" in spec.src
    assert spec.global_size == [2, 2, 1] and spec.local_size == [16, 16, 1]
    _compiles(spec)


def test_wmma_lowers_to_mfma():
    spec = U.render(KL.wmma_gemm_bf16(32, 32, 64), "w")
    assert "__builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0)" in spec.src
    assert "__WMMA_16_16_32_bfloat_float(" in spec.src
    assert spec.local_size == [64, 1, 1]
    _compiles(spec)
    k = KL.wmma_gemm_bf16(32, 32, 64)
    bad = [(n[0], n[1], n[2], n[3], n[4], n[5], n[6], "WMMA_8_8_8_float_float" if n[1] == U.WMMA else n[7], n[8])
           for n in k.nodes]
    k.nodes = bad
    with pytest.raises(MorokHipError) as e:
        U.render(k, "w")
    assert "no gfx950 MFMA lowering" in e.value.message


def test_local_memory_extension_ops_render():
    spec = U.render(KL.async_copy_transposing_load(), "tr")
    # a wave-uniform destination: M0 straight from a scalar expression, the source as the buffer's scalar
    # base plus the per-lane terms as a 32-bit offset
    assert "global_load_lds_dwordx4" in spec.src and "s_mov_b32 m0" in spec.src and '"s"(data1 + 0)' in spec.src
    assert 's_waitcnt vmcnt(0)' in spec.src
    assert "__builtin_amdgcn_ds_read_tr16_b64_v4bf16(" in spec.src
    morok_amd.compile_spec(spec)
    # a transposing load reads local memory, a direct copy goes from a PARAM to local memory
    k = U.Kernel()
    out = k.param(0, U.bf16, 256)
    inp = k.param(1, U.bf16, 512)
    k.store(k.index(out, k.const(0)), k.load_tr(k.index(inp, k.const(0))))
    with pytest.raises(morok_amd.MorokHipError):
        U.render(k, "bad_tr")
    k = U.Kernel()
    out = k.param(0, U.bf16, 256)
    inp = k.param(1, U.bf16, 512)
    k.async_copy(k.index(inp, k.const(0)), k.index(out, k.const(0)))
    with pytest.raises(morok_amd.MorokHipError):
        U.render(k, "bad_copy")


def test_wave_reduce_uses_dpp():
    spec = U.render(KL.wave_row_sum(8, 256), "wr")
    assert "__builtin_amdgcn_update_dpp" in spec.src and "__builtin_amdgcn_ds_swizzle" in spec.src
    assert "mrk_wave_reduce_add(" in spec.src
    _compiles(spec)


def test_variables_become_scalar_args():
    k = U.Kernel()
    out = k.param(0, U.f32, 1024)
    n = k.define_var("n", U.i32, 1, 1024)
    off = k.define_var("off", U.i64, 0, 1 << 40)
    l = k.special("lidx0", 256)
    g = k.special("gidx0", 4)
    idx = k.add(k.mul(g, k.const(256)), l)
    k.if_(k.binary("lt", idx, n))
    k.store(k.index(out, idx), k.cast(k.add(k.cast(idx, U.i64), off), U.f32))
    k.endif()
    spec = U.render(k, "v")
    assert "const int n, const long long off)" in spec.src
    assert spec.var_names == ["n", "off"]
    _compiles(spec)


def test_malformed_streams_are_rejected():
    with pytest.raises(MorokHipError):
        U.render(b"not a kernel", "x")
    k = KL.elementwise_unary("neg", 64)
    data = k.serialize()
    with pytest.raises(MorokHipError):
        U.render(data[: len(data) // 2], "x")
    k2 = U.Kernel()
    r = k2.range(4, 0)
    with pytest.raises(MorokHipError) as e:
        U.render(k2, "x")  # RANGE never closed
    assert "unbalanced" in e.value.message
    k3 = U.Kernel()
    k3.special("tidx0", 4)
    with pytest.raises(MorokHipError):
        U.render(k3, "x")
    k4 = U.Kernel()
    k4.special("lidx0", 2048)
    with pytest.raises(MorokHipError):
        U.render(k4, "x")
    k5 = U.Kernel()
    k5.param(0, U.f32, 4)
    k5.param(0, U.f32, 4)
    with pytest.raises(MorokHipError):
        U.render(k5, "x")
