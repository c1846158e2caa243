"""CPU-only checks of the C-ABI library: it loads, exports every symbol the public header
declares, and fails loudly (no fallback) where a GPU would be needed."""
import pytest

import morok_amd
from morok_amd import _ffi


def test_every_declared_symbol_is_exported_and_bound():
    declared = _ffi.declared_symbols()
    assert len(declared) > 40
    missing = [s for s in declared if not hasattr(_ffi.lib, s)]
    assert not missing, missing
    unbound = [s for s in declared if s not in _ffi._SIGS]
    assert not unbound, f"header declares symbols with no ctypes prototype: {unbound}"
    extra = [s for s in _ffi._SIGS if s not in declared]
    assert not extra, f"bound but not declared in the header: {extra}"


def test_device_spec_parse():
    # device/src/registry.rs:26-81 with the HIP arm
    assert morok_amd.parse_device("HIP") == 0
    assert morok_amd.parse_device("hip:3") == 3
    assert morok_amd.parse_device("GPU") == 0
    assert morok_amd.parse_device("amd:1") == 1
    for bad in ("CPU", "CUDA:0", "HIP:x", "HIP:", "", "DISK:/tmp/x"):
        with pytest.raises(morok_amd.MorokHipError) as e:
            morok_amd.parse_device(bad)
        assert e.value.code == 3  # MRK_ERR_INVALID_DEVICE
        assert "invalid device" in e.value.message


def test_names_and_cache_key():
    assert morok_amd.Device.base_device_key() == "HIP"
    assert morok_amd.cache_key() == "hip-gfx950"


def test_unknown_device_type_is_unsupported():
    import ctypes as C

    rc = _ffi.lib.mrk_hip_device_create_by_type(b"METAL", 0)
    assert rc == 13  # MRK_ERR_UNSUPPORTED_DEVICE, runtime/src/device_registry.rs:114-120
    assert b"unsupported device" in _ffi.lib.mrk_hip_last_error()
    assert isinstance(C.c_int(rc).value, int)


def test_compile_without_gpu_produces_code_object():
    # hiprtc cross-compiles for gfx950 without a device: AOT convention bytes != empty, src absent
    src = 'extern "C" __global__ void k(float* data0, const int n) { if ((int)threadIdx.x < n) data0[threadIdx.x] = 1.0f; }'
    spec = morok_amd.ProgramSpec.from_source("k", src, 1, ["n"], [0], (1, 1, 1), (64, 1, 1))
    assert spec.name == "k" and spec.buf_count == 1 and spec.var_names == ["n"]
    assert spec.global_size == [1, 1, 1] and spec.local_size == [64, 1, 1]
    c = morok_amd.compile_spec(spec)
    assert c.name == "k" and c.src is None
    assert c.bytes[:4] == b"\x7fELF" or len(c.bytes) > 1000


def test_compile_error_is_reported():
    spec = morok_amd.ProgramSpec.from_source("bad", "this is not HIP", 0)
    with pytest.raises(morok_amd.MorokHipError) as e:
        morok_amd.compile_spec(spec)
    assert e.value.code == 10 and "bad" in e.value.message


def test_workspace_queries_are_host_side_and_bounded():
    """The scratch sizes a caller asks about before it launches are pure functions of the shape (no device needed):
    zero where the product / attention needs none, whole slices otherwise, at most 16 MiB for attention."""
    from morok_amd._ffi import lib

    att = lib.mrk_hip_flash_attn_workspace_bytes
    # one to 32 queries, no causal rule, 256 keys and more: the key sequence may be split over workgroups
    assert att(1, 32, 1, 4096, 128, 0) == 6 * 32 * 16 * 130 * 4        # six key ranges, 32 pairs, 16 slots of 128 + 2 floats
    assert att(1, 32, 17, 4096, 128, 0) == 6 * 32 * 32 * 130 * 4       # from 17 queries on 32 slots a pair
    for args in ((1, 32, 1, 4096, 128, 1), (1, 32, 33, 4096, 128, 0), (1, 32, 1, 255, 128, 0), (1, 32, 1, 4096, 96, 0),
                 (0, 32, 1, 4096, 128, 0), (8, 32, 4096, 4096, 128, 1)):
        assert att(*args) == 0, args
    for b in (1, 2, 3, 7, 16, 64, 1000):
        for sq in (1, 4, 16, 32):
            for d in (64, 128, 256):
                for sk in (256, 1000, 4096, 1 << 17):
                    ws = att(b, 32, sq, sk, d, 0)
                    assert ws % ((d + 2) * 4 * 16) == 0 and ws <= 16 << 20, (b, sq, d, sk, ws)
    gemm = lib.mrk_hip_gemm_bf16_workspace_bytes
    assert gemm(4096, 4096, 4096, 1) == 0 and gemm(128, 4096, 11008, 1) > 0 and gemm(0, 4096, 4096, 1) == 0
