"""Scheduling helpers without a GPU: capability descriptor, tensor-core tables and the operand
layouts derived from them, GPU dimension limiting.  The gpudims cases restate the reference's
own unit tests (schedule/src/gpudims.rs:644-739); the layout checks pin the CDNA swizzle
tables (untested upstream) to the MFMA register layout measured on the hardware."""
import itertools
import random

import pytest

import morok_amd
from morok_amd import MorokHipError, sched, uop as U


def test_caps_match_reference_descriptor():
    c = sched.caps()  # schedule/src/optimizer/renderer.rs:290-303
    assert c["device"] == "AMD_CDNA4" and c["has_local"] == 1 and c["has_shared"] == 1 and c["has_threads"] == 0
    assert c["global_max"] == [2147483647, 65535, 65535] and c["local_max"] == 1024 and c["upcast_max"] == 8
    assert c["shared_max"] == 163840  # gfx950 LDS per workgroup (the reference lists 65536)
    # cdna4_tensor_cores(), renderer.rs:724-733: fp8e5m2, fp8e4m3, f16, bf16 (16x16x32), f16, bf16 (16x16x16);
    # the reference's WMMA name table has no entry for the 8-bit floats (tc.rs:677-688: "unknown")
    assert c["tensor_cores"][:6] == ["WMMA_16_16_32_unknown_float", "WMMA_16_16_32_unknown_float", "WMMA_16_16_32_half_float",
                                     "WMMA_16_16_32_bfloat_float", "WMMA_16_16_16_half_float", "WMMA_16_16_16_bfloat_float"]
    # behind them, two entries the reference does not have: the 32x32x16 shape of gfx950 (selection by dtype
    # still finds the reference's entries first)
    assert c["tensor_cores"][6:] == ["WMMA_32_32_16_half_float", "WMMA_32_32_16_bfloat_float"]


def test_tensor_core_selection():
    # tc.rs:126-168: first entry whose input and accumulator dtypes match
    assert sched.tc_select(U.BF16, U.BF16, U.F32) == 3
    assert sched.tc_select(U.F16, U.F16, U.F32) == 2
    assert sched.tc_select(U.FP8E5M2, U.FP8E5M2, U.F32) == 0
    assert sched.tc_select(U.FP8E4M3, U.FP8E4M3, U.F32) == 1
    assert sched.tc_select(U.FP8E4M3, U.FP8E5M2, U.F32) == -1
    assert sched.tc_select(U.F32, U.F32, U.F32) == -1
    assert sched.tc_select(U.BF16, U.BF16, U.BF16) == -1
    assert sched.tc_select(U.BF16, U.F16, U.F32) == -1
    dims, threads, ept = sched.tc_info(3)
    assert dims == [16, 16, 32] and threads == 64 and ept == [8, 8, 4]  # renderer.rs:549-558
    dims, threads, ept = sched.tc_info(5)
    assert dims == [16, 16, 16] and ept == [4, 4, 4]
    with pytest.raises(MorokHipError):
        sched.tc_info(11)
    dims, threads, ept = sched.tc_info(7)
    assert dims == [32, 32, 16] and threads == 64 and ept == [8, 8, 16]


@pytest.mark.parametrize("tc", [0, 1, 2, 3, 4, 5, 6, 7])
def test_swizzle_tables_equal_mfma_register_layout(tc):
    """Layout of v_mfma_f32_16x16x{16,32} and v_mfma_f32_32x32x16: with T the tile extent, lane l holds
    row/column l % T and the contiguous k group l // T of A/B; accumulator register e of lane l is
    C[(e // 4) * (256 // T) + 4 * (l // T) + e % 4][l % T] (16x16: 4 * (l // 16) + e).
    (The same formulas drive the one-hot MFMA test on the GPU.)"""
    (T, T2, K), _, (ea, eb, ec) = sched.tc_info(tc)
    per = K * T // 64
    assert T == T2 and ea == per and eb == per and ec == T * T // 64
    seen_a, seen_b, seen_c = set(), set(), set()
    for lane in range(64):
        for e in range(per):
            assert sched.tc_element(tc, 0, lane, e) == (lane % T, per * (lane // T) + e)
            assert sched.tc_element(tc, 1, lane, e) == (lane % T, per * (lane // T) + e)
            seen_a.add(sched.tc_element(tc, 0, lane, e))
            seen_b.add(sched.tc_element(tc, 1, lane, e))
        for e in range(ec):
            assert sched.tc_element(tc, 2, lane, e) == ((e // 4) * (256 // T) + 4 * (lane // T) + e % 4, lane % T)
            seen_c.add(sched.tc_element(tc, 2, lane, e))
    assert len(seen_a) == T * K and len(seen_b) == T * K and len(seen_c) == T * T  # every element exactly once


# ---- the reference's gpudims unit tests
def test_group_dims_cases():
    assert sched.group_dims([4, 4], [16, 16, 16]) == [4, 4]
    g = sched.group_dims([4, 4, 4, 4], [256, 256, 256])
    assert g is not None and len(g) <= 3 and g == [16, 4, 4]
    assert sched.group_dims([8, 8, 8], [256, 256, 256]) == [8, 8, 8]
    assert sched.group_dims([1000], [10]) is None


def test_split_dims_and_smallest_divisor():
    assert all(d <= 64 for d in sched.split_dims([100], [64, 64, 64]))
    assert sched.split_dims([100], [64, 64, 64]) == [50, 2]
    assert [sched.find_smallest_divisor(n) for n in (1, 2, 3, 4, 9, 100)] == [1, 2, 1, 2, 3, 2]


def test_get_contraction_cases():
    assert sched.get_contraction([2, 5, 2], [10, 2]) == [[0, 1], [2]]
    assert sched.get_contraction([4, 4, 4], [4, 4, 4]) == [[0], [1], [2]]
    assert sched.get_contraction([2, 3, 4], [24]) == [[0, 1, 2]]
    assert sched.get_contraction([2, 3, 4], [5, 4]) is None
    assert sched.get_contraction([2, 4, 3], [8, 3]) == [[0, 1], [2]]


def test_limit_dims_under_cdna4_limits():
    gmax = sched.caps()["global_max"]
    assert sched.limit_dims([8192, 8192], gmax) == [8192, 8192]
    assert sched.limit_dims([70000, 70000, 3, 5], gmax)[0] <= gmax[0]
    out = sched.limit_dims([4, 100000, 100000], gmax)  # y would exceed 65535: must be regrouped or split
    assert all(o <= m for o, m in zip(out, gmax)) and len(out) <= 3
    prod = 1
    for o in out:
        prod *= o
    assert prod == 4 * 100000 * 100000


def test_grouped_dims_index_mapping_is_a_bijection():
    """Integer/index work is bit-exact: every tuple of hardware indices maps to a distinct,
    in-range tuple of original indices, and all of them are covered."""
    rng = random.Random(7)
    cases = [([2, 5, 2], [16, 2]), ([6, 4], [8, 8, 8]), ([3, 3, 3, 3], [32, 32, 32]), ([100], [64, 64, 64]),
             ([7, 9], [63, 63]), ([12], [4, 4, 4])]
    for _ in range(20):
        n = rng.randint(1, 4)
        cases.append(([rng.choice([1, 2, 3, 4, 5, 6, 8]) for _ in range(n)], [rng.choice([8, 16, 64])] * 3))
    for dims, mx in cases:
        for reverse in (False, True):
            launch, _ = sched.grouped_dims(dims, mx, reverse)
            total = 1
            for d in dims:
                total *= d
            lt = 1
            for l in launch:
                lt *= l
            assert lt == total, (dims, mx, launch)
            seen = set()
            for raw in itertools.product(*[range(l) for l in launch]):
                _, idx = sched.grouped_dims(dims, mx, reverse, list(raw))
                assert all(0 <= i < d for i, d in zip(idx, dims)), (dims, launch, raw, idx)
                seen.add(tuple(idx))
            assert len(seen) == total, (dims, mx, reverse, launch)
    # global indices are assigned in reverse: the last (fastest) dimension gets gidx0
    launch, idx = sched.grouped_dims([3, 5], None, True, [4, 2])
    assert launch == [5, 3] and idx == [2, 4]
    launch, idx = sched.grouped_dims([3, 5], None, False, [2, 4])
    assert launch == [3, 5] and idx == [2, 4]


def test_matmul_kernels_render_and_compile():
    spec = U.render(sched.build_matmul_f32(128, 192, 64), "r_mm")
    assert spec.global_size == [3, 2, 1] and spec.local_size == [16, 16, 1] and "fmaf(" in spec.src
    morok_amd.compile_spec(spec)
    spec = U.render(sched.build_wmma_matmul(3, 64, 160, 128), "r_tc")
    # post-TC upcasts (heuristics.rs:787-821): M has 4 tiles -> upcast 4, N has 10 -> upcast 5
    assert spec.global_size == [2, 1, 1] and spec.local_size == [64, 1, 1]
    assert spec.src.count("__WMMA_16_16_32_bfloat_float(") == 20 + 1
    morok_amd.compile_spec(spec)
    with pytest.raises(MorokHipError) as e:
        sched.build_wmma_matmul(3, 60, 64, 64)
    assert "not a multiple" in e.value.message
    # the 8-bit-float cores: byte operands, eight per lane handed over as one 64-bit integer
    for tc, builtin in ((0, "__builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8"), (1, "__builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8")):
        spec8 = U.render(sched.build_wmma_matmul(tc, 32, 32, 64, U.F32), "r_tc8")
        assert builtin in spec8.src and "const unsigned char* __restrict__ data1" in spec8.src
        morok_amd.compile_spec(spec8)
        with pytest.raises(MorokHipError):
            sched.build_wmma_matmul_lds(tc, 128, 128, 64, U.F32)          # the LDS layouts are for 16-bit elements
    with pytest.raises(MorokHipError):                                    # an 8-bit-float result would need arithmetic on the carrier byte
        U.render(sched.build_wmma_matmul(1, 32, 32, 64, U.FP8E4M3), "r_tc8_out")
    morok_amd.compile_spec(U.render(sched.build_wmma_matmul(2, 32, 32, 64, U.F16), "r_tc16"))
    morok_amd.compile_spec(U.render(sched.build_wmma_matmul(4, 32, 32, 64, U.F32), "r_tc16k16"))


def test_wmma_matmul_lds_kernel_builds_and_compiles():
    """The LDS-staged tensor-core matmul renders to two __shared__ tiles, two barriers per K
    step and 16 MFMA builtins per wave and K step, and compiles for gfx950; shapes off the
    128 x 128 workgroup tile are refused."""
    import morok_amd
    from morok_amd import sched, uop as U

    kern = sched.build_wmma_matmul_lds(3, 256, 128, 64, U.BF16)
    spec = U.render(kern, "r_tc_lds")
    src = spec.src
    assert src.count("__shared__") == 2 and src.count("__syncthreads();") == 2
    assert "__builtin_amdgcn_mfma_f32_16x16x32_bf16" in src
    assert src.count("__WMMA_16_16_32_bfloat_float(") == 2 * 16 + 1   # two K steps x 4 x 4 tiles per wave + the definition
    assert spec.sizes() == ([1, 2, 1], [64, 4, 1])
    morok_amd.compile_spec(spec)
    assert "amdgpu_waves_per_eu(2)" in src                               # four waves, accumulators within half the file
    # extents the tile does not divide are padded: gated loads, guarded stores, a rounded-up grid
    pad = U.render(sched.build_wmma_matmul_lds(3, 200, 136, 72, U.BF16), "r_tc_pad")
    assert pad.sizes() == ([2, 2, 1], [64, 4, 1]) and " ? *((mrk_bhalf8*)" in pad.src and "if (" in pad.src
    morok_amd.compile_spec(pad)
    assert " ? *((mrk_bhalf8*)" not in src and "if (" not in src        # none of it when the tile divides
    with pytest.raises(morok_amd.MorokHipError):
        sched.build_wmma_matmul_lds(3, 64, 130, 64, U.BF16)               # rows of B are not whole 16-byte vectors


@pytest.mark.parametrize("opts,grid,block,mfma,hint", [((1, 1, 1, 1, 0), [8, 16, 1], [64, 1, 1], 2, False),
                                                       ((1, 4, 4, 1, 2), [2, 4, 1], [64, 4, 1], 8, True),
                                                       ((4, 2, 2, 4, 2), [1, 2, 1], [64, 8, 1], 16, True),
                                                       ((2, 2, 8, 4, 0), [1, 1, 1], [64, 4, 1], 64, False)])
def test_wmma_matmul_lds_kernel_choices(opts, grid, block, mfma, hint):
    """LOCAL (grid of waves), UPCAST (tiles per wave) and UNROLL (K steps per barrier pair) of
    the LDS-staged tensor-core kernel: launch dimensions and MFMA count follow the choices and
    every variant compiles; choices that do not divide the shape or the copies are refused."""
    import morok_amd
    from morok_amd import sched, uop as U

    M, N, K = 256, 128, 64
    spec = U.render(sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts), "r_tc_lds")
    assert spec.sizes() == (grid, block)
    assert spec.src.count("__WMMA_16_16_32_bfloat_float(") == mfma + 1
    # two waves per SIMD are asked for when four or more waves share a workgroup and the declared
    # registers (accumulators + copy staging) stay within 128 per work-item
    assert ("amdgpu_waves_per_eu(2)" in spec.src) == hint
    morok_amd.compile_spec(spec)


@pytest.mark.parametrize("opts", [(3, 2, 4, 4, 0), (2, 2, 4, 4, 3), (8, 8, 1, 1, 0), (2, 2, 8, 8, 0), (4, 4, 1, 1, 1),
                                  (2, 2, 4, 4, 8), (1, 1, 8, 8, 0)])
def test_wmma_matmul_lds_kernel_refuses_bad_choices(opts):
    import morok_amd
    from morok_amd import sched, uop as U

    with pytest.raises(morok_amd.MorokHipError):
        sched.build_wmma_matmul_lds_opts(3, 256, 128, 64, U.BF16, opts)


def test_wmma_matmul_direct_copy_kernel_builds_and_compiles():
    """stages = 2: both tiles in two stages of local memory filled by direct global -> local copies
    (extension ops ASYNC_COPY / WAIT_ASYNC), B fragments through the transposing load (LOAD_TR),
    one barrier per 64-deep K step plus the one that opens the loop and the one in front of the
    result staging, a flat grid whose workgroups are mapped to tiles per XCD; a 16-bit result is
    staged through the (then free) tile stages and written as 16-byte pieces, an f32 result as
    vectors of four straight from the accumulators."""
    import morok_amd
    from morok_amd import sched, uop as U

    M, N, K = 1024, 512, 256
    spec = U.render(sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, (2, 4, 8, 4, 0, 2)), "r_tc_dma")
    src = spec.src
    assert spec.sizes() == ([8, 1, 1], [64, 8, 1])                       # 4 x 2 tiles of 256 x 256, 8 waves
    assert "__shared__ __bf16 local0[32768];" in src and "__shared__ __bf16 local1[32768];" in src   # 2 stages x 256 x 64 each
    copies_per_wave = (256 // 8 + 256 // 8) // 8
    assert src.count("global_load_lds_dwordx4") == 3 * copies_per_wave    # tiles 0 and 1 up front, tile r + 2 in the loop
    assert src.count("__syncthreads();") == 3
    assert 's_waitcnt vmcnt(%d)' % copies_per_wave in src and src.count("s_waitcnt vmcnt(0)") == 1
    assert src.count("__builtin_amdgcn_ds_read_tr16_b64_v4bf16(") == 3 * 2 * 4   # 4 column tiles x (lo, hi) x (first half ahead, second, first)
    assert src.count("__WMMA_16_16_32_bfloat_float(") == 2 * 32 + 1
    assert "*((mrk_bhalf8*)((data0 +" in src and "*((mrk_bhalf4*)((data0 +" not in src   # 16-byte pieces of result rows
    f32_out = U.render(sched.build_wmma_matmul_lds_opts(3, M, N, K, U.F32, (2, 4, 8, 4, 0, 2)), "r_tc_dma_f32").src
    assert "*((mrk_float4*)((data0 +" in f32_out and f32_out.count("__syncthreads();") == 2
    assert "gidx0 % 8" in src                                              # the XCD regrouping
    morok_amd.compile_spec(spec)
    # a single K step has no loop-carried copies; half precision takes the f16 transposing load
    one = U.render(sched.build_wmma_matmul_lds_opts(3, 128, 128, 64, U.BF16, (2, 2, 4, 4, 0, 2)), "r_tc_dma1")
    assert one.src.count("global_load_lds_dwordx4") == (128 // 8 + 128 // 8) // 4 and "s_waitcnt vmcnt(0)" in one.src
    morok_amd.compile_spec(one)
    half = U.render(sched.build_wmma_matmul_lds_opts(2, 128, 128, 128, U.F16, (2, 2, 4, 4, 0, 2)), "r_tc_dma_h")
    assert "__builtin_amdgcn_ds_read_tr16_b64_v4f16(" in half.src
    morok_amd.compile_spec(half)
    # builtin form for the kernels above (their accumulators fit half of the register file)
    assert "__builtin_amdgcn_mfma_f32_16x16x32_bf16(" in src and "v_mfma_f32_16x16x32_bf16 %0" not in src


def test_wmma_matmul_direct_copy_one_wave_per_simd_is_written_out():
    """Four waves with 8 x 8 tiles each (256 accumulator registers, one wave per SIMD): the tensor-core
    instruction is written out with its accumulator tied in place in the accumulation registers,
    the waits the device compiler would insert around it are explicit (in front of the loop for the
    initial values, behind it for the last results, each followed by one empty statement per
    accumulator), every local-memory read and copy of the loop sits behind a tensor-core instruction
    of its own, and the loop has no branch (the last two steps copy the last tile again)."""
    import morok_amd
    from morok_amd import sched, uop as U

    M, N, K = 512, 512, 256
    spec = U.render(sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, (2, 2, 8, 8, 0, 2)), "r_tc_dma4")
    src = spec.src
    assert spec.sizes() == ([4, 1, 1], [64, 4, 1])
    assert 'asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));' in src
    assert "__builtin_amdgcn_mfma_f32_16x16x32_bf16(" not in src
    loop = src[src.index("for (int ridx0"):]
    loop = loop[:loop.index("\n  }\n")]
    # each trip of the loop holds two K steps (one per stage), so stage offsets are constants
    assert "ridx0 < 2;" in loop
    assert "if (" not in loop and loop.count("global_load_lds_dwordx4") == 32 and loop.count("__WMMA_16_16_32_bfloat_float(") == 256
    # no two reads or copies without a tensor-core instruction between them
    kinds = [("w" if "__WMMA_" in l else "m" if ("global_load_lds" in l or "ds_read_tr16" in l) else "") for l in loop.split("\n")]
    seq = "".join(kinds)
    assert "mmm" not in seq.replace("w", "|").replace("||", "|")  # (a B fragment is two transposing reads)
    before, after = src[:src.index("for (int ridx0")], src[src.index("for (int ridx0"):]
    assert before.count('asm volatile("" : "+a"(') == 64 and 'asm volatile("s_nop 7"' in before
    assert after.count('asm volatile("" : "+a"(') == 64 and after.count('asm volatile("s_nop 15"') == 2
    morok_amd.compile_spec(spec)
    half = U.render(sched.build_wmma_matmul_lds_opts(2, M, N, K, U.F16, (2, 2, 8, 8, 0, 2)), "r_tc_dma4_h")
    assert "v_mfma_f32_16x16x32_f16 %0" in half.src
    morok_amd.compile_spec(half)


def test_tc_matmul_direct_copy_refuses_what_it_cannot_tile():
    import morok_amd
    from morok_amd import sched, uop as U

    for shape, opts in (((500, 512, 256), (2, 2, 2, 2, 0, 2)),     # M is not a multiple of the tile
                        ((512, 512, 200), (2, 2, 2, 2, 0, 2)),     # K is not a multiple of 64
                        ((512, 512, 256), (2, 2, 2, 2, 1, 2)),     # the K step is 64 deep
                        ((512, 512, 256), (1, 1, 2, 2, 0, 2)),     # 32 columns: no whole granule group
                        ((1024, 1024, 256), (4, 4, 8, 8, 0, 2)),   # two stages of 512 x 512 exceed local memory
                        ((512, 512, 128), (2, 2, 2, 2, 0, 3)),     # three stages need more than two K steps
                        ((512, 512, 256), (2, 2, 2, 2, 0, 4))):    # no such variant
        with pytest.raises(morok_amd.MorokHipError):
            sched.build_wmma_matmul_lds_opts(3, *shape, U.BF16, opts)
    with pytest.raises(morok_amd.MorokHipError):
        sched.build_wmma_matmul_lds_opts(5, 512, 512, 256, U.BF16, (2, 2, 2, 2, 0, 2))   # a 16x16x16 tensor core


def test_global_index_order_modes_and_where_they_differ():
    """reverse=1 (dims reversed before limiting, indices after: what generated kernels launch) against
    reverse=2 (the literal code of schedule/src/gpudims.rs:331-382: only the index list is reversed).
    The two agree exactly on dims lists that read the same in both directions; on every other list
    mode 2 hands dimension i an index running over the extent of dimension n-1-i, so it is not an
    in-range bijection there."""
    GLOBAL_MAX = [2147483647, 65535, 65535]
    cases = [[7], [4, 4], [3, 5, 3], [3, 5], [2, 3, 4], [5, 1], [6, 6, 2], [2, 9, 9, 2], [2, 3, 3, 4], [70000, 4],
             [4, 70000], [70000, 70000], [3, 70000, 3]]
    for dims in cases:
        l1, _ = sched.grouped_dims(dims, GLOBAL_MAX, 1)
        l2, _ = sched.grouped_dims(dims, GLOBAL_MAX, 2)
        symmetric = dims == dims[::-1]
        total = 1
        for d in dims:
            total *= d
        if total > 5000:  # compare on a sample of hardware index tuples
            raws = [[min(r, l - 1) for l in l1] for r in (0, 1, 2, 69999)]
        else:
            raws = [list(r) for r in itertools.product(*[range(l) for l in l1])]
        if symmetric:
            assert l1 == l2, dims
            for raw in raws:
                assert sched.grouped_dims(dims, GLOBAL_MAX, 1, raw)[1] == sched.grouped_dims(dims, GLOBAL_MAX, 2, raw)[1]
        else:
            # mode 1 stays in range for every tuple; mode 2 leaves it for some tuple
            out_of_range = False
            for raw in itertools.product(*[range(min(l, 6)) for l in l2]):
                _, idx = sched.grouped_dims(dims, GLOBAL_MAX, 2, list(raw))
                out_of_range = out_of_range or any(i >= d for i, d in zip(idx, dims))
            for raw in raws:
                _, idx = sched.grouped_dims(dims, GLOBAL_MAX, 1, raw)
                assert all(0 <= i < d for i, d in zip(idx, dims)), (dims, raw, idx)
            assert out_of_range or l1 != l2, dims
    # the innermost axis is gidx0 in mode 1 whatever regrouping happened
    assert sched.grouped_dims([3, 5], GLOBAL_MAX, 1)[0] == [5, 3]
    assert sched.grouped_dims([3, 5], GLOBAL_MAX, 2)[0] == [3, 5]
    assert sched.grouped_dims([70000, 4], GLOBAL_MAX, 1)[0] == [280000]          # y would exceed 65535: grouped
    assert sched.grouped_dims([70000, 4], GLOBAL_MAX, 1, [9])[1] == [2, 1]        # 9 = 2 * 4 + 1
    assert sched.grouped_dims([2, 3, 70000, 8], GLOBAL_MAX, 1)[0] == [560000, 3, 2]
    with pytest.raises(Exception):
        sched.grouped_dims([3, 5], GLOBAL_MAX, 3)
