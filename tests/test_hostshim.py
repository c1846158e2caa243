"""Host runtime logic without a GPU: the product's host sources run against host-memory
stand-ins for the HIP layer (tests/hostshim).  Covers what a GPU run cannot force (device
out-of-memory -> LRU clear + retry) and everything that is pure host logic: lazy allocation,
views, size checks, launch-dimension conventions, kernel cache, the lowering of lazy tensor
graphs into kernels (counts, names, fused-kernel selection, rendered source compiles)."""
import ctypes as C

import numpy as np
import pytest

import morok_amd
from morok_amd import MorokHipError, uop
from tests import hostshim_lib


@pytest.fixture()
def shim(monkeypatch):
    lib = hostshim_lib.load()
    import morok_amd._ffi as f
    import morok_amd.device as d
    import morok_amd.ops as o
    import morok_amd.sched as s
    import morok_amd.tensor as t

    for mod in (f, d, o, s, t, uop, morok_amd):
        if hasattr(mod, "lib"):
            monkeypatch.setattr(mod, "lib", lib)
    lib.mrk_shim_reset()
    lib.mrk_hip_tensor_set_fusion(1)
    yield lib
    lib.mrk_shim_reset()


@pytest.fixture()
def dev(shim):
    d = morok_amd.Device("HIP")
    d.lru_clear()
    return d


# ------------------------------------------------------------------ device / allocator
def test_shim_is_not_the_product_library(shim):
    assert shim._name.endswith("libmorok_hostshim.so")
    assert morok_amd._ffi.LIB_PATH.endswith("libmorok_hip.so")


def test_invalid_device_ordinal(shim):
    with pytest.raises(MorokHipError) as e:
        morok_amd.Device("HIP:3")
    assert e.value.code == 3  # InvalidDevice (device/src/error.rs)


def test_lru_reuse_and_limits(dev, shim):
    p = dev.alloc(4096)
    calls = shim.mrk_shim_alloc_calls()
    dev.free(p, 4096)
    assert dev.lru_cache_count(4096) == 1 and shim.mrk_shim_free_calls() == 0  # cached, not freed
    assert dev.alloc(4096) == p and shim.mrk_shim_alloc_calls() == calls     # reuse without a device call
    dev.free(p, 4096)
    ptrs = [dev.alloc(512) for _ in range(40)]
    for x in ptrs:
        dev.free(x, 512)
    assert dev.lru_cache_count(512) == 32          # allocator.rs: at most 32 per key
    assert shim.mrk_shim_free_calls() == 8         # the overflow went back to the device
    dev.lru_clear()
    assert dev.lru_total_cached() == 0 and shim.mrk_shim_bytes_in_use() == 0


def test_zero_init_on_reuse(dev, shim):
    p = dev.alloc(1000)
    junk = np.full(1000, 0xAB, np.uint8)
    morok_amd._ffi.check(shim.mrk_hip_copyin(0, p, 0, junk.ctypes.data_as(C.c_void_p), 1000))
    dev.free(p, 1000)
    q = dev.alloc(1000, zero_init=True)
    assert q == p
    out = np.empty(1000, np.uint8)
    morok_amd._ffi.check(shim.mrk_hip_copyout(0, out.ctypes.data_as(C.c_void_p), q, 0, 1000))
    assert not out.any()
    # fresh (non-reused) memory with zero_init is zeroed too; without it the content is arbitrary
    r = dev.alloc(2000, zero_init=True)
    out = np.empty(2000, np.uint8)
    morok_amd._ffi.check(shim.mrk_hip_copyout(0, out.ctypes.data_as(C.c_void_p), r, 0, 2000))
    assert not out.any()
    dev.free(q, 1000)
    dev.free(r, 2000)


def test_allocator_properties(dev, shim):
    """device/src/test/proptests.rs restated with hypothesis over random sizes and flags:
    a freed block is reused for any later request of the same (size, cpu_accessible) key and
    of no other; a buffer and its views cache exactly one block when both are gone; a reused
    block requested with zero_init comes back zeroed; the cache never holds more than 32
    blocks per key whatever the order of allocations and frees."""
    from hypothesis import given, settings, HealthCheck, strategies as st

    sizes = st.integers(min_value=1, max_value=1 << 16)

    @settings(max_examples=60, deadline=None, suppress_health_check=list(HealthCheck))
    @given(size=sizes, other=sizes, cpu=st.booleans(), other_cpu=st.booleans())
    def reuse_by_key(size, other, cpu, other_cpu):
        dev.lru_clear()
        p = dev.alloc(size, cpu_accessible=cpu)
        dev.free(p, size, cpu_accessible=cpu)
        assert dev.lru_cache_count(size, cpu) == 1
        q = dev.alloc(other, cpu_accessible=other_cpu)
        same_key = other == size and other_cpu == cpu
        assert (q == p) == same_key
        assert dev.lru_cache_count(size, cpu) == (0 if same_key else 1)
        dev.free(q, other, cpu_accessible=other_cpu)

    @settings(max_examples=40, deadline=None, suppress_health_check=list(HealthCheck))
    @given(size=st.integers(min_value=20, max_value=1 << 16), zero=st.booleans())
    def views_and_zero_init(size, zero):
        dev.lru_clear()
        b = morok_amd.Buffer(size)
        b.ensure_allocated()
        v = b.view(0, min(size, 10))
        assert v.id == b.id
        junk = np.full(size, 0x5A, np.uint8)
        b.copyin(junk)
        del v, b
        assert dev.lru_cache_count(size) == 1           # one block for the buffer and its view together
        b2 = morok_amd.Buffer(size, zero_init=zero)
        b2.ensure_allocated()
        assert dev.lru_cache_count(size) == 0           # reused
        got = b2.copyout(np.uint8, (size,))
        assert (not got.any()) if zero else np.all(got == 0x5A)
        del b2

    @settings(max_examples=15, deadline=None, suppress_health_check=list(HealthCheck))
    @given(ops=st.lists(st.tuples(st.sampled_from([64, 4096, 65536]), st.booleans()), min_size=1, max_size=120))
    def capacity(ops):
        dev.lru_clear()
        live = []
        for size, do_free in ops:
            if do_free and live:
                p, sz = live.pop()
                dev.free(p, sz)
            else:
                live.append((dev.alloc(size), size))
            for sz in (64, 4096, 65536):
                assert dev.lru_cache_count(sz) <= 32
        many = [dev.alloc(64) for _ in range(50)]
        for p in many:
            dev.free(p, 64)
        assert dev.lru_cache_count(64) == 32
        for p, sz in live:
            dev.free(p, sz)

    reuse_by_key()
    views_and_zero_init()
    capacity()
    dev.lru_clear()
    assert shim.mrk_shim_bytes_in_use() == 0


def test_out_of_memory_clears_cache_and_retries(dev, shim):
    """allocator.rs:173-190: on an allocation failure the LRU frees everything it holds and
    retries once; only a second failure is reported."""
    shim.mrk_shim_set_memory_limit(10_000)
    a = dev.alloc(6000)
    dev.free(a, 6000)                      # 6000 bytes now sit in the cache
    assert shim.mrk_shim_bytes_in_use() == 6000
    b = dev.alloc(7000)                    # 6000 + 7000 > limit: must clear the cache, then succeed
    assert shim.mrk_shim_bytes_in_use() == 7000 and dev.lru_total_cached() == 0
    with pytest.raises(MorokHipError) as e:
        dev.alloc(5000)                    # nothing left to clear: the error surfaces
    assert e.value.code == 8 and "hipErrorOutOfMemory" in str(e.value)
    dev.free(b, 7000)
    c = dev.alloc(5000)                    # works again once memory came back
    dev.free(c, 5000)


# ------------------------------------------------------------------ buffers
def test_buffer_lazy_views_and_size_checks(dev, shim):
    before = shim.mrk_shim_alloc_calls()
    b = dev.buffer(64)
    assert not b.is_allocated() and shim.mrk_shim_alloc_calls() == before   # buffer.rs: lazy
    data = np.arange(16, dtype=np.float32)
    b.copyin(data)
    assert b.is_allocated()
    v = b.view(16, 32)
    assert v.id == b.id                                                     # views share the id
    np.testing.assert_array_equal(v.copyout(np.float32), data[4:12])
    with pytest.raises(MorokHipError) as e:
        b.copyin(np.zeros(3, np.float32))
    assert e.value.code == 1                                                # SizeMismatch
    with pytest.raises(MorokHipError) as e:
        b.view(48, 32)
    assert e.value.code == 6                                                # InvalidView
    other = dev.buffer(64)
    other.copy_from(b)
    np.testing.assert_array_equal(other.copyout(np.float32), data)
    with pytest.raises(MorokHipError):
        dev.buffer(32).copy_from(b)
    b.release()
    assert dev.lru_cache_count(64) == 0   # the view still holds the allocation
    v.release()
    assert dev.lru_cache_count(64) == 1


# ------------------------------------------------------------------ compile / launch plumbing
SRC = """extern "C" __global__ void scale(float* out, const float* in, const int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) out[i] = in[i] * 2.0f; }"""


def test_compile_load_launch_dimensions(dev, shim):
    spec = morok_amd.ProgramSpec.from_source("scale", SRC, 2, var_names=["n"], global_size=(5, 2, 1), local_size=(64, 1, 1))
    comp = morok_amd.compile_spec(spec)
    assert comp.bytes[:4] == b"\x7fELF"
    prog = morok_amd.Program.create(comp)
    a, b = dev.buffer(1024).ensure_allocated(), dev.buffer(1024).ensure_allocated()
    n = shim.mrk_shim_launches()
    prog.execute([a, b], [256])
    assert shim.mrk_shim_launches() == n + 1 and shim.mrk_shim_last_kernel() == b"scale"
    # global_size counts workgroups, local_size is the workgroup shape
    assert hostshim_lib.last_dims(shim) == ((5, 2, 1), (64, 1, 1))
    prog.execute([a, b], [256], global_size=(7, 1, 1), local_size=(32, 2, 1))
    assert hostshim_lib.last_dims(shim) == ((7, 1, 1), (32, 2, 1))
    with pytest.raises(MorokHipError):
        prog.execute([a], [256])          # wrong buffer count
    with pytest.raises(MorokHipError):
        prog.execute([a, b], [])          # wrong variable count


def test_missing_entry_point_and_compile_error(dev, shim):
    spec = morok_amd.ProgramSpec.from_source("nope", SRC, 2, var_names=["n"], global_size=(1, 1, 1), local_size=(1, 1, 1))
    with pytest.raises(MorokHipError) as e:
        morok_amd.Program.create(morok_amd.compile_spec(spec))
    assert "nope" in str(e.value)
    bad = morok_amd.ProgramSpec.from_source("k", "extern \"C\" __global__ void k(float* o) { o[0] = undefined_symbol; }", 1,
                                            global_size=(1, 1, 1), local_size=(1, 1, 1))
    with pytest.raises(MorokHipError) as e:
        morok_amd.compile_spec(bad)
    assert e.value.code == 10 and "undefined_symbol" in str(e.value)


# ------------------------------------------------------------------ lazy tensor lowering
@pytest.fixture()
def T(dev):
    from morok_amd import tensor

    return tensor


def zeros(T, shape, dtype=np.float32, tag=None):
    return T.Tensor.from_numpy(np.zeros(shape, dtype), tag)


def test_tensor_shapes_and_errors(T):
    t = zeros(T, (2, 3, 4))
    assert t.try_permute([2, 0, 1]).shape == (4, 2, 3)
    assert t.try_reshape([6, -1]).shape == (6, 4)
    assert t.sum(1).shape == (2, 4) and t.sum(1, keepdim=True).shape == (2, 1, 4)
    assert t.try_add(zeros(T, (4,))).shape == (2, 3, 4)
    assert t.matmul(zeros(T, (4, 5))).shape == (2, 3, 5)
    assert zeros(T, (7, 8)).embedding(zeros(T, (2, 3), np.int32)).shape == (2, 3, 8)
    assert t.binary("lt", 1.0).dtype == uop.BOOL
    assert zeros(T, (4,), np.uint16, uop.BF16).try_add(zeros(T, (4,))).dtype == uop.F32
    assert zeros(T, (4,), np.uint16, uop.BF16).rms_norm(-1, 1e-6).dtype == uop.F32
    for bad in (lambda: t.try_reshape([5, 5]), lambda: t.try_permute([0, 0, 1]), lambda: t.try_add(zeros(T, (5,))),
                lambda: t.try_expand([2, 3, 5]), lambda: t.try_shrink([(0, 3), (0, 3), (0, 4)]),
                lambda: t.matmul(zeros(T, (3, 4))), lambda: t.softmax(3)):
        with pytest.raises(MorokHipError) as e:
            bad()
        assert e.value.code == 11
    with pytest.raises(MorokHipError) as e:
        T.Tensor.from_bytes(b"\0" * 10, (3,), uop.F32)
    assert e.value.code == 1 and "data length 10 != expected 12" in str(e.value)


def test_tensor_kernel_counts_generated(T, shim):
    T.set_fusion(False)
    s = zeros(T, (8, 300)).softmax(-1).realize()
    assert len(s.kernels()) == 3                     # max, sum, divide (fusion.rs:83-88)
    assert [k[0] for k in s.kernels()] == ["r", "r", "E"]
    m = zeros(T, (96, 40)).matmul(zeros(T, (40, 24))).realize()
    assert len(m.kernels()) == 1                     # fusion.rs:28-33
    r = zeros(T, (64, 8192)).rms_norm(-1, 1e-6).realize()
    assert len(r.kernels()) == 2                     # mean-of-squares reduce + scale (too few rows for one workgroup per row to fill the chip)
    r = zeros(T, (4, 512)).rms_norm(-1, 1e-6).realize()
    assert r.kernels() == ["rE_4_g512_4"]            # a handful of short rows is bound by launches: one row-resident kernel
    e = zeros(T, (16, 8)).embedding(zeros(T, (3,), np.int32)).try_mul(2.0).realize()
    assert len(e.kernels()) == 1                     # the gather fuses into its consumer
    x = zeros(T, (2, 4, 6, 8))
    rope = x.apply_rotary_emb(zeros(T, (1, 1, 6, 4)), zeros(T, (1, 1, 6, 4)), False).realize()
    assert len(rope.kernels()) == 1
    rope_i = x.apply_rotary_emb(zeros(T, (1, 1, 6, 4)), zeros(T, (1, 1, 6, 4)), True).realize()
    assert len(rope_i.kernels()) == 1
    # a cat of computed halves on the innermost axis becomes one guarded region per half, with
    # the work-items renumbered so that a wave stays inside one half
    xr = zeros(T, (2, 16, 4, 128))
    big = xr.apply_rotary_emb(zeros(T, (1, 16, 1, 64)), zeros(T, (1, 16, 1, 64)), False).realize()
    src = T.last_kernel_sources()[0]
    assert len(big.kernels()) == 1 and src.count("if (") == 3 and " ? " not in src.split("if (", 2)[2]
    # interleaved pairs: the reshape [.., 128] -> [.., 64, 2] splits the upcast group; positions along
    # the trailing axis stay compile-time constants, so nothing is selected and x is one vector load
    inter = xr.apply_rotary_emb(zeros(T, (1, 16, 1, 64)), zeros(T, (1, 16, 1, 64)), True).realize()
    src = T.last_kernel_sources()[0]
    assert len(inter.kernels()) == 1 and " ? " not in src and src.count("*((mrk_float4*)") == 2   # the load of x, the store
    small = x.apply_rotary_emb(zeros(T, (1, 1, 6, 4)), zeros(T, (1, 1, 6, 4)), False).realize()
    assert T.last_kernel_sources()[0].count("if (") == 1          # too few outputs for whole waves: select as before
    assert len(small.kernels()) == 1
    a = x.scaled_dot_product_attention(x, x, is_causal=True).realize()
    assert len(a.kernels()) == 4                     # QK^T, max, sum, PV (the divide fuses into PV)
    sw = zeros(T, (1000,)).silu().realize()
    assert len(sw.kernels()) == 1


def test_tensor_fused_kernel_selection(T, shim):
    s = zeros(T, (8, 300)).softmax(-1).realize()
    assert s.kernels() == ["softmax_f32"] or (len(s.kernels()) == 1 and s.kernels()[0].startswith("softmax"))
    assert shim.mrk_shim_last_kernel() == b"softmax_f32"
    s2 = zeros(T, (8, 300)).softmax(0).realize()
    assert len(s2.kernels()) == 3                    # not the last axis: generated kernels
    bf = lambda *shape: zeros(T, shape, np.uint16, uop.BF16)
    g = bf(64, 32).matmul(bf(32, 48)).realize()
    assert len(g.kernels()) == 1 and shim.mrk_shim_last_kernel() == b"gemm_bf16"
    f = bf(1, 2, 64, 128).scaled_dot_product_attention(bf(1, 2, 64, 128), bf(1, 2, 64, 128), is_causal=True).realize()
    assert len(f.kernels()) == 1 and shim.mrk_shim_last_kernel() == b"flash_fwd_bf16"
    f64 = bf(1, 2, 64, 64).scaled_dot_product_attention(bf(1, 2, 64, 64), bf(1, 2, 64, 64), is_causal=True).realize()
    assert f64.kernels() == ["flash_fwd_bf16_2_64_64_d64"]   # head dim 64 has an instantiation of its own
    f256 = bf(1, 2, 64, 256).scaled_dot_product_attention(bf(1, 2, 64, 256), bf(1, 2, 64, 256), is_causal=True).realize()
    assert f256.kernels() == ["flash_fwd_bf16_2_64_64_d256"]  # and so has 256
    # one query against a long key sequence with few (batch, head) pairs: the key sequence is split over workgroups
    # and the kernel gets a scratch buffer for the ranges' partial results, an intermediate of the plan
    dec = bf(1, 8, 1, 128).scaled_dot_product_attention(bf(1, 8, 2048, 128), bf(1, 8, 2048, 128)).realize()
    assert dec.kernels() == ["flash_fwd_bf16_8_1_2048_splitkv"] and shim.mrk_shim_last_kernel() == b"flash_fwd_bf16_splitkv"
    dec_c = bf(1, 8, 1, 128).scaled_dot_product_attention(bf(1, 8, 2048, 128), bf(1, 8, 2048, 128), is_causal=True).realize()
    assert dec_c.kernels() == ["flash_fwd_bf16_8_1_2048"]    # not under the causal rule
    f96 = bf(1, 2, 64, 96).scaled_dot_product_attention(bf(1, 2, 64, 96), bf(1, 2, 64, 96), is_causal=True).realize()
    # other head dims are padded with zero columns to the next instantiation: three padded copies, the
    # fused kernel at 128, the cut back to 96 columns; no reduce kernels, no score matrix
    assert sum(k.startswith("flash_fwd_bf16_2_64_64") for k in f96.kernels()) == 1 and not any(k.startswith("r_") for k in f96.kernels())
    f300 = bf(1, 2, 64, 304).scaled_dot_product_attention(bf(1, 2, 64, 304), bf(1, 2, 64, 304), is_causal=True).realize()
    assert len(f300.kernels()) >= 4 and any(k.startswith("r_") for k in f300.kernels())   # beyond 256: the composed graph
    m = zeros(T, (128, 40)).matmul(zeros(T, (40, 64))).realize()
    assert len(m.kernels()) == 1 and m.kernels()[0] == "r_128_64_40"  # scheduled f32 matmul
    h = zeros(T, (256, 128), np.float16).matmul(zeros(T, (128, 192), np.float16)).realize()
    assert h.kernels() == ["gemm_f16_256_192_128"] and shim.mrk_shim_last_kernel() == b"gemm_f16"     # half: hand-written too
    hw = zeros(T, (192, 128), np.float16)
    assert zeros(T, (512, 128), np.float16).linear(hw).realize().kernels() == ["gemm_f16_nt_512_192_128"]
    T.set_fusion(False)
    h = zeros(T, (256, 128), np.float16).matmul(zeros(T, (128, 192), np.float16)).realize()
    assert h.kernels() == ["r_tc_256_192_128"] and "mfma_f32_16x16x32_f16" in T.last_kernel_sources()[0]   # switched off: the WMMA route
    T.set_fusion(True)
    # inputs that are lazy views get materialised first
    gt = bf(32, 64).try_transpose(0, 1).matmul(bf(32, 48)).realize()
    assert len(gt.kernels()) == 2


def test_tensor_kernel_cache_and_realize_idempotent(T, shim):
    from morok_amd import tensor

    morok_amd.kernel_cache_clear()
    a = zeros(T, (1000,)).try_mul(3.0).try_add(1.0).realize()
    assert tensor.last_cached_count() == 0
    size = morok_amd.kernel_cache_size()
    b = zeros(T, (1000,)).try_mul(3.0).try_add(1.0).realize()
    assert tensor.last_cached_count() == 1 and morok_amd.kernel_cache_size() == size
    n = shim.mrk_shim_launches()
    b.realize()
    assert shim.mrk_shim_launches() == n and tensor.last_kernels() == []
    c = zeros(T, (1001,)).try_mul(3.0).try_add(1.0).realize()   # other shape, other kernel
    assert tensor.last_cached_count() == 0 and morok_amd.kernel_cache_size() == size + 1
    assert a.shape == (1000,) and c.shape == (1001,)


def test_tensor_launch_dims_come_from_grouped_dims(T, shim):
    """Generated kernels take their grid from get_grouped_dims under the device limits
    (schedule/src/gpudims.rs:331-382, global_max [2147483647, 65535, 65535]): rows x workgroups-per-row
    as (x = innermost, y = rows) while rows fit y, regrouped into x beyond that."""
    T.set_fusion(False)
    zeros(T, (300, 1024)).try_add(1.0).realize()          # 256 work-items tile a row of 1024 / 4 exactly
    assert hostshim_lib.last_dims(shim) == ((1, 300, 1), (256, 1, 1))
    zeros(T, (300, 4096)).try_add(1.0).realize()
    assert hostshim_lib.last_dims(shim) == ((4, 300, 1), (256, 1, 1))
    zeros(T, (70000, 1024)).try_add(1.0).realize()        # 70000 rows exceed 65535 in y: grouped into x
    assert hostshim_lib.last_dims(shim) == ((70000, 1, 1), (256, 1, 1))
    src = T.last_kernel_sources()[0]
    assert "blockIdx.y" not in src
    zeros(T, (70000, 2048)).try_add(1.0).realize()
    assert hostshim_lib.last_dims(shim) == ((140000, 1, 1), (256, 1, 1))
    zeros(T, (2, 3, 5, 1024)).try_add(1.0).realize()      # leading axes count as rows
    assert hostshim_lib.last_dims(shim) == ((1, 30, 1), (256, 1, 1))
    zeros(T, (300, 1000)).try_add(1.0).realize()          # rows the workgroups do not tile: flat
    assert hostshim_lib.last_dims(shim) == ((293, 1, 1), (256, 1, 1))


def test_tensor_launch_dims(T, shim):
    T.set_fusion(False)
    zeros(T, (1001,)).try_add(1.0).realize()
    assert hostshim_lib.last_dims(shim) == ((4, 1, 1), (256, 1, 1))
    zeros(T, (8, 1000)).try_add(1.0).realize()      # innermost axis % 4 == 0: four outputs per work-item
    assert hostshim_lib.last_dims(shim) == ((8, 1, 1), (256, 1, 1))
    zeros(T, (10, 4096)).sum(1).realize()           # few outputs: eight wavefronts share each through local memory
    assert hostshim_lib.last_dims(shim) == ((10, 1, 1), (64, 8, 1))
    zeros(T, (5000, 4096)).sum(1).realize()         # many outputs: one wavefront per output, four per workgroup
    assert hostshim_lib.last_dims(shim) == ((1250, 1, 1), (64, 4, 1))
    zeros(T, (100, 16)).sum(1).realize()            # short rows: one work-item per output
    assert hostshim_lib.last_dims(shim) == ((2, 1, 1), (64, 1, 1))


@pytest.mark.parametrize("tag,npdt", [("U8", np.uint8), ("I8", np.int8), ("I16", np.int16), ("U16", np.uint16)])
def test_narrow_integer_kernels_compile(T, shim, tag, npdt):
    """Vectorised kernels on 8- and 16-bit integers: the promoted-to-int arithmetic must be cast
    back inside vector literals for the source to compile."""
    dt = getattr(uop, tag)
    x = T.Tensor.from_numpy(np.zeros((4, 64), npdt), dt)
    y = x.try_add(T.Tensor.const(3, dt)).try_mul(x)
    y.realize()
    assert len(y.kernels()) == 1 and y.dtype == dt


def test_tensor_int64_indexing_for_huge_views(T, shim):
    """A broadcast view with more than 2^31 elements feeding a reduce must index in 64 bits."""
    T.set_fusion(False)
    t = T.Tensor.full([1 << 16, 1 << 16], 1.0, uop.F32).sum(1)
    t.realize()
    # 65536 inputs per output: two-stage reduction; both generated sources compiled
    assert len(t.kernels()) == 2


@pytest.mark.parametrize("fused,gemms", [(True, 4), (False, 7)])
def test_decoder_block_lowering(T, shim, fused, gemms):
    """The decoder block graph lowers to 7 GEMMs (4 with Wq|Wk|Wv and W1|W3 stored side by
    side) + 1 flash attention + the generated elementwise / reduce kernels; weights and tokens
    never reach a real device here."""
    from morok_amd import decoder, synth

    cfg = dict(batch=2, seq=64, hidden=256, heads=2, ffn=512)
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], 100, seed=1)
    blk = decoder.DecoderBlock(w, cfg["batch"], cfg["seq"], cfg["hidden"], cfg["heads"], cfg["ffn"],
                               fuse_projections=fused)
    n0 = shim.mrk_shim_launches()
    out = blk.forward(T.Tensor.from_numpy(synth.randint((128,), 1, 1, 100))).realize()
    names = out.kernels()
    assert out.shape == (128, 256) and out.dtype == uop.BF16
    assert sum(k.startswith("gemm_bf16") for k in names) == gemms
    assert sum(k.startswith("flash_fwd") for k in names) == 1
    assert shim.mrk_shim_launches() - n0 == len(names)
    # the attention kernel writes [tokens, hidden] itself and reads V in place out of the
    # projection's [tokens, ...] result: neither is copied into [batch, heads, seq, dim]
    assert sum(k.startswith("flash_fwd_bf16_strided") for k in names) == 1
    # both residual additions happen in the epilogue of the product in front of them
    assert sum(k.startswith("gemm_bf16_residual") for k in names) == 2
    # with gate and up stored side by side, silu(gate) * up happens in the epilogue of their product
    assert sum(k.startswith("gemm_bf16_swiglu") for k in names) == (1 if fused else 0)
    # fused: q | k are rotated in the epilogue of the packed QKV product (no rotary kernel of its own)
    assert sum(k.startswith("gemm_bf16_rope") for k in names) == (1 if fused else 0)
    assert len(names) == (10 if fused else 16)


def test_decoder_block_first_norm_writes_the_embedding_rows(T, shim):
    """With rows wide enough for the row-resident kernel (hidden 512: 64 work-items of 8 elements),
    the embedding lookup the caller asked to have in memory (`contiguous()`, the residual reads it
    later) is computed by the first RMSNorm kernel itself and written as that kernel's second
    output: 7 kernels in all (norm, QKV + rotary, attention, Wo + residual, norm, gated product,
    W2 + residual); switched off, the lookup is a kernel of its own again."""
    import os

    from morok_amd import decoder, synth

    cfg = dict(batch=2, seq=64, hidden=512, heads=4, ffn=1024)
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], 100, seed=1)

    def lower():
        blk = decoder.DecoderBlock(w, cfg["batch"], cfg["seq"], cfg["hidden"], cfg["heads"], cfg["ffn"])
        return blk.forward(T.Tensor.from_numpy(synth.randint((128,), 1, 1, 100))).realize().kernels()

    names = lower()
    assert len(names) == 7, names
    assert names[0] == "rE_128_g512_8_s1" and sum(k.startswith("rE_128_g512_8") for k in names) == 2
    assert not any(k.startswith("E_") for k in names)
    os.environ["MOROK_NO_SIDE_OUTPUTS"] = "1"
    try:
        names = lower()
    finally:
        del os.environ["MOROK_NO_SIDE_OUTPUTS"]
    assert len(names) == 8 and names[0].startswith("E_") and names[1] == "rE_128_g512_8"


def test_linear_layout_weights_are_read_in_place(T, shim):
    """x @ w.T with w [out, in] in memory (tensor/src/nn/linear.rs:39-41): the product kernels
    take the weight as it is stored instead of a transposed copy, also under the residual and the
    gated epilogue; shapes those kernels do not cover copy the transpose as before."""
    bf = lambda shape: zeros(T, shape, np.uint16, uop.BF16)
    x, w = bf((512, 256)), bf((768, 256))
    y = x.linear(w)
    assert y.shape == (512, 768) and y.realize().kernels() == ["gemm_bf16_nt_512_768_256"]
    # the same through an explicit transpose, and with a bias (added in the product kernel's epilogue; a bias that
    # is an expression, or a product with a second reader, is added by a kernel of its own)
    assert x.matmul(w.try_transpose(0, 1)).realize().kernels() == ["gemm_bf16_nt_512_768_256"]
    assert x.linear(w, bf((768,))).realize().kernels() == ["gemm_bf16_nt_bias_512_768_256"]
    assert x.matmul(bf((256, 768))).try_add(bf((768,))).realize().kernels() == ["gemm_bf16_bias_512_768_256"]
    names = x.linear(w, bf((768,)).try_mul(2.0).cast(uop.BF16)).realize().kernels()
    assert names[0] == "gemm_bf16_nt_512_768_256" and len(names) == 2
    p = x.linear(w)
    names = p.try_add(bf((768,))).try_mul(p).realize().kernels()
    assert names[0] == "gemm_bf16_nt_512_768_256" and len(names) == 2
    # residual epilogue
    h = bf((512, 768))
    assert h.try_add(x.linear(w)).realize().kernels() == ["gemm_bf16_nt_residual_512_768_256"]
    # gated epilogue over a [2F, K] weight
    w13 = bf((2 * 384, 256))
    gu = x.linear(w13)
    g = gu.try_shrink([(0, 512), (0, 384)]).silu().try_mul(gu.try_shrink([(0, 512), (384, 768)]))
    assert g.realize().kernels() == ["gemm_bf16_nt_swiglu_512_384_256"]
    # a weight that is not in memory as such (an expression) is computed in the layout the kernel reads
    names = x.matmul(w.try_mul(2.0).cast(uop.BF16).try_transpose(0, 1)).realize().kernels()
    assert names[-1] == "gemm_bf16_512_768_256" and len(names) == 2
    # with fusion off nothing is matched
    T.set_fusion(False)
    try:
        assert not any(k.startswith("gemm_bf16") for k in x.linear(w).realize().kernels())
    finally:
        T.set_fusion(True)


def test_plan_graph_replay_records_once(T, shim):
    """execute_graph records the plan's launches once (nothing runs while recording), replays
    them with one graph launch per call, and drops the recording when variables are rebound or
    the plan goes away."""
    x = T.Tensor.from_numpy(np.arange(64, dtype=np.float32).reshape(8, 8))
    y = x.try_add(x).sum([1]).try_exp()      # a reduce and an elementwise kernel
    plan = y.prepare()
    n = plan.kernel_count
    assert n >= 2
    base = shim.mrk_shim_launches()
    plan.execute()
    assert shim.mrk_shim_launches() - base == n
    plan.execute_graph()                      # records n launches, then one graph launch runs them
    assert shim.mrk_shim_launches() - base == 2 * n and shim.mrk_shim_graph_launches() == 1
    assert shim.mrk_shim_graphs_alive() == 1
    plan.execute_graph()
    plan.execute_graph()
    assert shim.mrk_shim_launches() - base == 4 * n and shim.mrk_shim_graph_launches() == 3
    plan.execute_with_vars({})                # rebinding drops the recording
    assert shim.mrk_shim_graphs_alive() == 0
    plan.execute_graph()
    assert shim.mrk_shim_graphs_alive() == 1
    del plan
    import gc

    gc.collect()
    assert shim.mrk_shim_graphs_alive() == 0


# ------------------------------------------------------------------ beam-search support
def test_beam_cache_roundtrip_and_ignore(shim, tmp_path, monkeypatch):
    from morok_amd import sched

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)
    assert sched.beam_cache_get(1234, 4, "HIP:0") is None
    sched.beam_cache_put(1234, 4, "HIP:0", b"\x01\x02\x03")
    assert sched.beam_cache_get(1234, 4, "HIP:0") == b"\x01\x02\x03"
    # the key covers the AST hash, the beam width and the device (beam.rs:401-409)
    assert sched.beam_cache_get(1234, 8, "HIP:0") is None
    assert sched.beam_cache_get(1234, 4, "HIP:1") is None
    assert sched.beam_cache_get(1235, 4, "HIP:0") is None
    sched.beam_cache_put(1234, 4, "HIP:0", b"new")          # overwrite
    assert sched.beam_cache_get(1234, 4, "HIP:0") == b"new"
    assert (tmp_path / "beam_cache_hip").is_dir()
    monkeypatch.setenv("IGNORE_BEAM_CACHE", "1")             # beam.rs:16-19
    assert sched.beam_cache_get(1234, 4, "HIP:0") is None


def test_compile_and_time_and_failing_candidates(dev, shim):
    from morok_amd import sched

    bufs = [dev.buffer(64 * 64 * 4) for _ in range(3)]
    k = sched.build_matmul_f32_opts(64, 64, 64, [16, 16, 4, 4, 2])
    n = shim.mrk_shim_launches()
    ms = sched.compile_and_time(k, bufs, warmup=1, runs=3)
    assert ms >= 0.0 and shim.mrk_shim_launches() == n + 4           # 1 warm-up + 3 timed launches
    assert hostshim_lib.last_dims(shim) == ((1, 1, 1), (16, 16, 1))
    with pytest.raises(MorokHipError):                                # wrong buffer count: a status, not a crash
        sched.compile_and_time(k, bufs[:2])
    with pytest.raises(MorokHipError) as e:                           # choices that do not divide the shape
        sched.build_matmul_f32_opts(64, 64, 64, [16, 16, 4, 8, 1])
    assert e.value.code == 11
    with pytest.raises(MorokHipError):
        sched.compile_and_time(b"not a kernel", bufs)


def test_beam_search_over_generated_kernels(dev, shim, tmp_path, monkeypatch):
    """MOROK_BEAM also searches the generated elementwise and reduce kernels: candidates are built
    like the real kernel, compiled and timed; the winner is cached on disk under the hash of the
    heuristic kernel, so a second realization of the same graph compiles and times nothing; small
    kernels are left to the heuristics; the kernel list keeps its shape."""
    from morok_amd import tensor as T

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)

    def graph():
        a = T.Tensor.from_numpy(np.ones((512, 1024), np.float32))
        b = T.Tensor.from_numpy(np.ones((512, 1024), np.float32))
        return a.try_add(b).try_exp().sum(-1)

    graph().realize()
    plain = T.last_kernels()
    assert T.last_beam_search() == (0, 0)
    monkeypatch.setenv("MOROK_BEAM", "2")
    graph().realize()
    timed, hits = T.last_beam_search()
    assert timed >= 4 and hits == 0
    assert len(T.last_kernels()) == len(plain)
    graph().realize()
    assert T.last_beam_search() == (0, 1)
    # elementwise: UPCAST and LOCAL candidates; tiny kernels are not searched
    big = T.Tensor.from_numpy(np.ones((256, 2048), np.float32))
    big.try_mul(big).cast(uop.BF16).realize()
    timed, hits = T.last_beam_search()
    assert timed >= 6 and hits == 0 and T.last_kernels()[0].startswith("E_524288")
    small = T.Tensor.from_numpy(np.ones((16, 16), np.float32))
    small.try_mul(small).realize()
    assert T.last_beam_search() == (0, 0)
    # a row-resident kernel: the work-items per row are searched
    rows = T.Tensor.from_numpy(np.ones((256, 4096), np.float32))
    rows.rms_norm(-1, 1e-6).realize()
    timed, hits = T.last_beam_search()
    assert timed >= 3 and hits == 0 and T.last_kernels() == ["rE_256_g4096_4"]


def test_row_resident_fusion_needs_a_path_that_keeps_the_row(T):
    """A keepdim reduction reaches the fused kernel's consumer as the workgroup's own row total,
    so it may only be fused when every path to it keeps the row coordinate: a transpose, a
    shrink or a reshape that moves the reduced axis in between must keep the separate kernel."""
    def names(t):
        t.realize()
        return T.last_kernels()

    x = zeros(T, (256, 256))
    same_row = x.try_add(x.sum(1, keepdim=True).try_expand([256, 256]))
    assert names(same_row) == ["rE_256_g256_4"]
    squeezed = x.try_mul(x.sum(1).try_reshape([256, 1]).try_expand([256, 256]))      # drop and re-add the axis of extent 1
    assert names(squeezed) == ["rE_256_g256_4"]
    other_row = x.try_add(x.sum(1, keepdim=True).try_transpose(0, 1).try_expand([256, 256]))   # x[i, j] + rowsum[j]
    assert not any(k.startswith("rE_") for k in names(other_row)) and len(T.last_kernels()) == 2
    as_columns = x.try_add(x.sum(1).try_reshape([1, 256]).try_expand([256, 256]))
    assert not any(k.startswith("rE_") for k in names(as_columns))
    b = zeros(T, (128, 128, 64))
    batch_swapped = b.try_add(b.sum(2, keepdim=True).try_permute([1, 0, 2]).try_expand([128, 128, 64]))
    assert not any(k.startswith("rE_") for k in names(batch_swapped))
    y = zeros(T, (512, 256))
    shifted = y.try_shrink([(0, 256), (0, 256)]).try_add(y.sum(1, keepdim=True).try_shrink([(256, 512), (0, 1)]).try_expand([256, 256]))
    assert not any(k.startswith("rE_") for k in names(shifted))
    # the second reduction of a chain must keep the row as well
    m = x.max(1, keepdim=True)
    chain = x.try_sub(m.try_transpose(0, 1).try_expand([256, 256])).try_exp()
    bad_chain = chain.try_div(chain.sum(1, keepdim=True).try_expand([256, 256]))
    assert not any(k.endswith("_x2") for k in names(bad_chain))
    good = names(zeros(T, (256, 1024), np.uint16, uop.BF16).softmax(-1))
    assert len(good) == 1 and good[0].startswith("rE_") and good[0].endswith("_x2")


def test_beam_search_uses_and_fills_the_disk_cache(dev, shim, tmp_path, monkeypatch):
    from morok_amd import sched

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)
    opts, ms, cached, timed = sched.beam_search_matmul_f32(128, 128, 64, width=2)
    assert not cached and timed > 10 and len(opts) == 6 and opts[5] in (0, 8, 16, 32)
    assert 128 % (opts[0] * opts[2]) == 0 and 128 % (opts[1] * opts[3]) == 0 and 64 % opts[4] == 0
    opts2, _, cached2, timed2 = sched.beam_search_matmul_f32(128, 128, 64, width=2)
    assert cached2 and timed2 == 0 and opts2 == opts
    _, _, cached3, _ = sched.beam_search_matmul_f32(128, 128, 64, width=3)    # other width, other key
    assert not cached3
    # odd shapes fall back to scalar columns / single rows instead of failing
    opts4, _, _, _ = sched.beam_search_matmul_f32(6, 10, 7, width=1)
    assert 10 % (opts4[0] * opts4[2]) == 0 and 6 % (opts4[1] * opts4[3]) == 0


# ------------------------------------------------------------------ hardware queues
def test_queue_batches_until_submit_and_reports_errors(dev, shim):
    k = morok_amd.Kernel.get_or_compile(__import__("morok_amd").sched.build_matmul_f32_opts(64, 64, 64, [16, 16, 4, 4, 1]), "qk")
    a, b, c = (dev.buffer(64 * 64 * 4) for _ in range(3))
    sig = morok_amd.TimelineSignal()
    q = morok_amd.HardwareQueue()
    n = shim.mrk_shim_launches()
    q.exec(k, [c, a, b]).signal(sig, 1).memory_barrier()
    assert q.pending == 2 and shim.mrk_shim_launches() == n        # nothing reaches the device before submit
    q.submit().synchronize()
    assert q.pending == 0 and shim.mrk_shim_launches() == n + 1 and sig.value == 1
    # a copy between buffers of different sizes is refused at submit (buffer.rs:411-534)
    q.copy(dev.buffer(16), dev.buffer(32))
    with pytest.raises(MorokHipError) as e:
        q.submit()
    assert e.value.code == 1 and q.pending == 0
    # waiting on a value nobody signals times out instead of hanging
    q2 = morok_amd.HardwareQueue(copy_queue=True)
    q2.wait(sig, 5)
    with pytest.raises(MorokHipError) as e:
        q2.submit(wait_timeout_ms=20)
    assert e.value.code == 12
    q2.wait(sig, 1).copy(a, b).submit(wait_timeout_ms=20)          # already reached: no wait


def test_queue_orders_against_the_device_stream_and_keeps_buffers_alive(dev, shim):
    """A zero_init buffer's fill is queued on the device stream when the buffer is first
    allocated (here: inside submit); the queue's stream must wait for the device stream before the
    kernel that writes the buffer.  The buffers of a batch stay referenced until the batch has
    completed, and the device stream waits for the batch before their blocks can be reused."""
    k = morok_amd.Kernel.get_or_compile(__import__("morok_amd").sched.build_matmul_f32_opts(64, 64, 64, [16, 16, 4, 4, 1]), "qk")
    nbytes = 64 * 64 * 4 + 4096                     # a size nothing else in this test uses
    a, b = dev.buffer(nbytes), dev.buffer(nbytes)
    a.ensure_allocated(), b.ensure_allocated()
    c = dev.buffer(nbytes, zero_init=True)          # lazy: allocated (and zero-filled) at submit
    q = morok_amd.HardwareQueue()
    shim.mrk_shim_set_events_pending(1)             # the GPU has not finished anything yet
    shim.mrk_shim_trace(1)
    q.exec(k, [c, a, b]).submit()
    ops = hostshim_lib.trace(shim)
    fill = next(i for i, o in enumerate(ops) if o.startswith("memset:"))
    dev_stream = ops[fill].split(":")[1]
    rec = next(i for i, o in enumerate(ops) if o.startswith("record:") and o.endswith(":" + dev_stream) and i > fill)
    ev = ops[rec].split(":")[1]
    launch = next(i for i, o in enumerate(ops) if o.startswith("launch:"))
    q_stream = ops[launch].split(":")[1]
    assert q_stream != dev_stream
    assert fill < rec < ops.index(f"wait:{q_stream}:{ev}") < launch, ops
    # the caller lets go of its buffer right after submit: the block is not recycled yet
    before = dev.lru_cache_count(nbytes)
    del c
    assert dev.lru_cache_count(nbytes) == before
    q.exec(k, [a, a, b]).submit()                   # a later submit does not retire an unfinished batch
    assert dev.lru_cache_count(nbytes) == before
    shim.mrk_shim_trace(1)
    shim.mrk_shim_set_events_pending(0)
    q.synchronize()                                 # now it has run: the block goes back to the cache,
    assert dev.lru_cache_count(nbytes) == before + 1
    ops = hostshim_lib.trace(shim)                  # and the device stream was told to wait for the batch
    assert any(o.startswith(f"wait:{dev_stream}:") for o in ops), ops


def test_memory_planner_reuses_intermediates(T, shim, monkeypatch):
    """tensor/src/memory_planner.rs: intermediates with disjoint lifetimes share blocks; outputs
    and inputs never do."""
    from morok_amd import decoder, synth, tensor

    cfg = dict(batch=2, seq=64, hidden=256, heads=2, ffn=512)
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], 100, seed=1)
    blk = decoder.DecoderBlock(w, cfg["batch"], cfg["seq"], cfg["hidden"], cfg["heads"], cfg["ffn"])
    tok = T.Tensor.from_numpy(synth.randint((128,), 1, 1, 100))
    dev = morok_amd.Device("HIP")
    dev.lru_clear()
    base = shim.mrk_shim_bytes_in_use()
    out = blk.forward(tok).realize()
    reused, saved = tensor.last_memory_plan()
    pool_bytes = tensor.last_intermediate_bytes()
    planned_bytes = shim.mrk_shim_bytes_in_use() - base
    assert reused >= 4 and saved >= 3 * 128 * 256 * 2
    del out
    dev.lru_clear()
    monkeypatch.setenv("MOROK_NO_MEMORY_PLANNER", "1")
    base = shim.mrk_shim_bytes_in_use()
    out2 = blk.forward(tok).realize()
    assert tensor.last_memory_plan() == (0, 0)
    unplanned_bytes = shim.mrk_shim_bytes_in_use() - base
    assert planned_bytes < unplanned_bytes and unplanned_bytes - planned_bytes >= saved // 2
    assert tensor.last_intermediate_bytes() == pool_bytes + saved       # one block per intermediate
    del out2


def test_planned_intermediates_become_lazy_again(T, shim):
    x = zeros(T, (64, 64))
    mid = x.try_add(1.0).contiguous()              # an intermediate of the first realization
    a = mid.try_mul(2.0).sum(1).realize()
    assert len(a.kernels()) == 2
    b = mid.try_mul(3.0).realize()                 # mid's block may have been reused: it is recomputed
    assert len(b.kernels()) == 2
    c = a.try_add(1.0).realize()                   # a was an output: it is read, not recomputed
    assert len(c.kernels()) == 1


def test_failed_schedule_leaves_the_graph_lazy(T, shim):
    """A kernel that fails to load in the middle of a realization must not leave provisional
    buffers on the nodes scheduled before it: the next realization of the same graph has to
    schedule (and launch) every kernel again instead of reading never-computed memory."""
    T.set_fusion(False)
    morok_amd.kernel_cache_clear()
    x = zeros(T, (37, 53))
    mid = x.try_add(1.0).sum(1)                    # kernel 1 (reduce)
    root = mid.try_mul(2.0).contiguous().sum(0)    # kernels 2 and 3
    shim.mrk_shim_fail_module_load_after(1)        # the second kernel's code object is refused
    n = shim.mrk_shim_launches()
    with pytest.raises(MorokHipError):
        root.realize()
    assert shim.mrk_shim_launches() == n           # nothing ran
    with pytest.raises(MorokHipError):             # extraction does not hand out an unrealised root either
        shim.mrk_shim_fail_module_load_after(0)
        root.to_numpy()
    root.realize()                                 # now everything loads
    assert len(root.kernels()) == 3 and shim.mrk_shim_launches() == n + 3
    again = mid.try_mul(3.0).realize()             # the shared reduce is scheduled again, not read
    assert len(again.kernels()) == 2


# ------------------------------------------------------------------ Tensor::to / COPY items
def test_host_tensors_and_lazy_device_copies(T, shim):
    """tensor/src/realize.rs:1322-1347 (device of from_slice, to() on the same / another device) and
    realize.rs:1002-1011 (COPY as an item of the plan, executed in order with the kernels)."""
    T.set_fusion(False)
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    allocs = shim.mrk_shim_alloc_calls()
    shim.mrk_shim_trace(1)
    a = T.Tensor.from_slice(x)
    assert a.device == "CPU" and a.shape == (3, 4)          # from_slice defaults to the CPU device
    assert a.to("CPU").device == "CPU" and a.to("cpu").to_numpy().tolist() == x.tolist()
    b = a.to("HIP:0")
    assert b.device == "HIP:0" and a.device == "CPU"        # the source stays where it was
    assert T.Tensor.from_slice_with(x, device="HIP").device == "HIP:0"
    # lazy: neither creation nor to() allocated device memory or moved a byte
    assert shim.mrk_shim_alloc_calls() == allocs and hostshim_lib.trace(shim) == []
    b.realize()
    assert b.kernels() == ["copy_h2d_48"] and hostshim_lib.trace(shim).count("htod:0") == 1
    assert b.to_numpy().tolist() == x.tolist()
    # a computation over the copy: the copy item precedes the kernel in the same plan
    shim.mrk_shim_trace(1)
    c = T.Tensor.from_slice(x).to("HIP:0").try_mul(2.0)
    plan = c.prepare()
    assert [plan.kernel_name(i) for i in range(plan.kernel_count)] == ["copy_h2d_48", "E_12_4"]
    assert "htod:0" not in hostshim_lib.trace(shim)          # deferred to execute time
    plan.execute()
    plan.execute()
    ops = hostshim_lib.trace(shim)
    assert ops.count("htod:0") == 2 and ops.index("htod:0") < ops.index("launch:0")
    with pytest.raises(MorokHipError) as e:                   # copies are not graph nodes
        plan.execute_graph()
    assert "copy" in str(e.value)
    # device -> CPU as the last step, and the whole round trip in one plan
    back = T.Tensor.from_slice(x).to("HIP:0").to("CPU")
    assert back.device == "CPU"
    assert back.to_numpy().tolist() == x.tolist() and back.kernels() == ["copy_h2d_48", "copy_d2h_48"]
    n = shim.mrk_shim_launches()
    assert back.as_vec().tolist() == x.ravel().tolist() and shim.mrk_shim_launches() == n  # realized once
    assert back.to("HIP:0").realize().kernels() == ["copy_h2d_48"]      # host bytes of a copy can go up again
    # a reshape of stored host bytes is the same bytes
    assert T.Tensor.from_slice(x).try_reshape([4, 3]).to("HIP:0").to_numpy().tolist() == x.reshape(4, 3).tolist()


def test_host_tensor_errors(T, shim):
    x = np.ones((4,), np.float32)
    cpu = T.Tensor.from_slice(x)
    for bad in (lambda: cpu.try_add(1.0).realize(),                       # no CPU compute in this backend
                lambda: cpu.try_add(1.0).to("HIP:0").realize(),           # not stored bytes
                lambda: cpu.try_add(T.Tensor.from_numpy(x)).realize(),    # operand left on the CPU
                lambda: T.Tensor.from_numpy(x).to("CPU").to("HIP:0").try_add(cpu.to("HIP:0").to("CPU")).realize()):
        with pytest.raises(MorokHipError) as e:
            bad()
        assert e.value.code == 13, str(e.value)                            # UnsupportedDevice
    with pytest.raises(MorokHipError) as e:
        cpu.to("HIP:5")
    assert e.value.code == 3
    with pytest.raises(MorokHipError):
        cpu.to("TPU:0")
    with pytest.raises(MorokHipError) as e:
        T.Tensor.from_slice(np.zeros(3, np.float32)).to_numpy().shape and lib_check_size(T)
    assert e.value.code == 1
    # a failed realization leaves the graph lazy (no half-made host buffers)
    t = T.Tensor.from_numpy(x).try_add(1.0).to("CPU")
    shim.mrk_shim_fail_module_load_after(0)
    morok_amd.kernel_cache_clear()
    with pytest.raises(MorokHipError):
        t.realize()
    assert t.to_numpy().shape == (4,)


def lib_check_size(T):
    from morok_amd._ffi import check, lib

    t = T.Tensor.from_slice(np.zeros(3, np.float32))
    out = np.empty(2, np.float32)
    check(lib.mrk_hip_tensor_to_bytes(t._h, out.ctypes.data_as(C.c_void_p), out.nbytes))


def test_ops_refuse_undersized_buffers(dev, shim):
    from morok_amd import ops

    small, big = dev.buffer(1024), dev.buffer(64 * 64 * 4)
    n = shim.mrk_shim_launches()
    with pytest.raises(ValueError):
        ops.softmax_f32(small, big, 64, 64)
    with pytest.raises(ValueError):
        ops.gemm_bf16(big, big, small, 64, 64, 64)
    with pytest.raises(ValueError):
        ops.flash_attn_fwd_bf16(big, big, small, big, 1, 1, 64, 64, 128, 0.1)
    with pytest.raises(ValueError):
        ops.fill_normal(small, 1 << 20)
    assert shim.mrk_shim_launches() == n             # nothing was launched
    ops.softmax_f32(big, big, 64, 64)
    assert shim.mrk_shim_last_kernel() == b"softmax_f32"


def test_flash_attention_refuses_heads_whose_rows_pass_4_gib(dev, shim):
    """The attention kernels form row offsets inside one (batch, head) in 32 bits: a dense head
    of 512-byte rows (head_dim 256) holds at most 2^23 - 1 rows, one of 256-byte rows 2^24 - 1; a strided
    operand's last row must end below 4 GiB as well.  Refused before anything is launched."""
    n = shim.mrk_shim_launches()
    one = C.c_void_p(16)
    rows = 1 << 23
    assert shim.mrk_hip_flash_attn_fwd_bf16(0, one, one, one, one, 1, 1, 128, rows, 256, C.c_float(1.0), 0) == 11
    assert b"4 GiB" in shim.mrk_hip_last_error()
    assert shim.mrk_hip_flash_attn_fwd_bf16(0, one, one, one, one, 1, 1, rows, 128, 256, C.c_float(1.0), 0) == 11
    assert shim.mrk_hip_flash_attn_fwd_bf16(0, one, one, one, one, 1, 1, 128, rows - 1, 256, C.c_float(1.0), 0) == 0
    assert shim.mrk_hip_flash_attn_fwd_bf16(0, one, one, one, one, 1, 1, 128, rows, 128, C.c_float(1.0), 0) == 0
    st = (C.c_int64 * 12)(*([0, 0, 128] * 4))
    st[5] = 1 << 20                                   # key rows 2 MiB apart: 4096 of them pass 4 GiB
    assert shim.mrk_hip_flash_attn_fwd_bf16_strided(0, one, one, one, one, 1, 1, 128, 4096, 128, C.c_float(1.0), 0, st) == 11
    assert b"operand 1" in shim.mrk_hip_last_error()
    assert shim.mrk_hip_flash_attn_fwd_bf16_strided(0, one, one, one, one, 1, 1, 128, 2048, 128, C.c_float(1.0), 0, st) == 0
    assert shim.mrk_shim_launches() == n + 3


def test_tensor_from_buffer_view_alignment(T, dev):
    b = dev.buffer(1024).ensure_allocated()
    t = T.Tensor.from_buffer(b.view(64, 256), (64,), uop.F32)
    assert t.shape == (64,)
    with pytest.raises(MorokHipError) as e:
        T.Tensor.from_buffer(b.view(4, 256), (64,), uop.F32)
    assert e.value.code == 11
    with pytest.raises(MorokHipError) as e:
        T.Tensor.from_buffer(b, (100,), uop.F32)
    assert e.value.code == 1


def test_large_reductions_are_split_in_two_stages(T, shim):
    """split_reduceop (schedule/src/rangeify/kernel.rs:44-61): >= 32768 inputs per output."""
    T.set_fusion(False)
    t = zeros(T, (1 << 20,)).sum(0).realize()
    # 256 waves as 16 workgroups of 16: the waves of a workgroup meet in local memory, 16 partials are left
    assert t.kernels() == ["r_1x16_g65536_l16", "r_1_16"]
    assert hostshim_lib.last_dims(shim) == ((1, 1, 1), (64, 1, 1))
    t = zeros(T, (4, 70000)).max(1).realize()        # few outputs: 16 waves share each, no second kernel
    assert t.kernels() == ["r_4_g70000_l16"]
    t = zeros(T, (4096, 70000)).max(1).realize()     # many outputs: split as before
    assert len(t.kernels()) == 2
    t = zeros(T, (64, 4096)).sum(1).realize()        # below the threshold: one kernel
    assert len(t.kernels()) == 1


def test_column_reductions_and_flat_upcast_lowering(T, shim):
    """Reductions that keep the contiguous axis run a work-item per output (split over the outermost
    reduce axis when the outputs alone are too few); elementwise kernels over an innermost axis that
    does not divide into 16-byte groups walk the output flat.  Every source compiles."""
    T.set_fusion(False)
    t = zeros(T, (8192, 4096)).max(0).realize()
    assert t.kernels() == ["r_4096x64_128", "r_4096_64"]
    assert all("global_load_lds" not in s and "__shared__" not in s for s in T.last_kernel_sources())
    t = zeros(T, (129, 64)).sum(0).realize()             # an odd reduce extent is not split
    assert t.kernels() == ["r_64_129"]
    t = zeros(T, (4, 2048, 256)).sum(1).realize()        # a fold over a middle axis
    assert len(t.kernels()) == 2 and t.kernels()[0].startswith("r_1024x")
    t = zeros(T, (64, 8192)).sum(1).realize()            # the innermost axis is reduced: waves along the rows, as before
    assert t.kernels() == ["r_64_g8192_l16"]
    a, b = zeros(T, (1000, 333)), zeros(T, (1000, 333))
    t = a.try_mul(b).try_add(a).realize()
    assert t.kernels() == ["E_333000_4f"]
    src = T.last_kernel_sources()[0]
    assert src.count("*((mrk_float4*)") == 3              # two vector loads and the vector store
    t = a.try_add(zeros(T, (1, 333)).try_expand([1000, 333])).realize()
    assert t.kernels() == ["E_333000_4f"] and T.last_kernel_sources()[0].count("*((mrk_float4*)") == 2   # the broadcast row stays scalar
    t = zeros(T, (333, 1000)).try_permute([1, 0]).contiguous().realize()
    assert t.kernels() == ["E_333000"]                    # nothing to read flat: the scalar walk


def test_grouped_reduce_through_local_memory(T, shim, monkeypatch):
    """GROUP / GROUPTOP (schedule/src/optimizer/heuristics.rs:370-392): kernels with at most 2048
    outputs let the waves of a workgroup share an output through local memory and a barrier."""
    T.set_fusion(False)
    t = zeros(T, (64, 8192)).sum(1).realize()
    assert t.kernels() == ["r_64_g8192_l16"]         # 16 waves per output, one launch
    assert hostshim_lib.last_dims(shim) == ((64, 1, 1), (64, 16, 1))
    src = T.last_kernel_sources()[0]
    assert "__shared__ float local0[16]" in src and "__syncthreads()" in src
    t = zeros(T, (512, 2048)).max(1).realize()       # more outputs: fewer waves each
    assert t.kernels() == ["r_512_g2048_l4"]
    t = zeros(T, (2048, 1024)).max(1).realize()      # enough outputs to fill the chip by themselves
    assert t.kernels() == ["r_2048_g1024"]
    t = zeros(T, (4096, 4096)).sum(1).realize()      # many outputs: one wave per output as before
    assert t.kernels() == ["r_4096_g4096"]
    t = zeros(T, (8, 300)).sum(1).realize()          # short rows: nothing to share
    assert t.kernels() == ["r_8_g300"]
    t = zeros(T, (8, 1 << 20)).sum(1).realize()      # split: the first stage leaves 16 partials per output
    assert t.kernels() == ["r_8x16_g65536_l16", "r_8_16"]
    t = zeros(T, (256, 65536)).sum(1).realize()      # 16 waves per output already cover the chip: one launch
    assert t.kernels() == ["r_256_g65536_l16"]
    monkeypatch.setenv("MOROK_NO_GROUP_REDUCE", "1")
    morok_amd.kernel_cache_clear()
    t = zeros(T, (64, 8192)).sum(1).realize()
    assert t.kernels() == ["r_64_g8192"]


def test_null_arguments_are_errors_not_crashes(T, dev, shim):
    """Every entry point checks its pointers: a null handle or output slot yields
    MRK_ERR_INVALID_ARGUMENT with a message, never a fault in the library."""
    import ctypes as C

    x = zeros(T, (4, 4))
    out = C.c_void_p()
    null = None
    calls = [
        lambda: shim.mrk_hip_tensor_sdpa_ex(null, x._h, x._h, null, 0.0, 0, 0.0, C.byref(out)),
        lambda: shim.mrk_hip_tensor_sdpa_ex(x._h, null, x._h, null, 0.0, 0, 0.0, C.byref(out)),
        lambda: shim.mrk_hip_tensor_sdpa_ex(x._h, x._h, x._h, null, 0.0, 0, 0.0, null),
        lambda: shim.mrk_hip_tensor_tanh(null, C.byref(out)),
        lambda: shim.mrk_hip_tensor_tanh(x._h, null),
        lambda: shim.mrk_hip_tensor_matmul_with(x._h, null, -1, C.byref(out)),
        lambda: shim.mrk_hip_tensor_matmul_with(x._h, x._h, 99, C.byref(out)),
        lambda: shim.mrk_hip_tensor_gemm(x._h, null, 1.0, 1.0, 0, 0, null, C.byref(out)),
        lambda: shim.mrk_hip_tensor_linear(x._h, null, null, -1, C.byref(out)),
        lambda: shim.mrk_hip_tensor_linear(x._h, x._h, null, 99, C.byref(out)),
        lambda: shim.mrk_hip_tensor_log_softmax(null, -1, C.byref(out)),
        lambda: shim.mrk_hip_tensor_logsumexp(x._h, -1, null),
        lambda: shim.mrk_hip_gemm_bf16_residual(0, null, 1, 1, 1, 8, 8, 8),
        lambda: shim.mrk_hip_flash_attn_fwd_bf16_strided(0, 1, 1, 1, 1, 1, 1, 8, 8, 128, 1.0, 0, null),
        lambda: shim.mrk_hip_sched_build_wmma_matmul_lds_opts(3, 128, 128, 64, 10, null, C.byref(C.POINTER(C.c_uint8)()), C.byref(C.c_size_t())),
        lambda: shim.mrk_hip_beam_search_wmma_matmul(2, 1, 128, 128, 64, 1, null, null, null, null),
        lambda: shim.mrk_hip_benchmark_kernel_with_cutoff(0, null, null, 0, null, 0, null, null, 1, 1, 0.0, null, null, null),
    ]
    for i, call in enumerate(calls):
        rc = call()
        assert rc == 11, (i, rc, shim.mrk_hip_last_error())       # MRK_ERR_INVALID_ARGUMENT
        assert shim.mrk_hip_last_error()
