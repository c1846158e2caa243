"""Device boundary on the GPU: allocator + LRU cache, Buffer views and copies, compile ->
program -> execute, error behaviour.  Mirrors the reference's device tests
(device/src/test/unit/buffer.rs, device/src/buffer.rs:580-602, device/src/allocator.rs:366-429)."""
import numpy as np
import pytest

import morok_amd
from morok_amd import MorokHipError

pytestmark = pytest.mark.gpu


def test_device_factory_and_registry(dev):
    assert morok_amd.device_count() >= 1
    d2 = morok_amd.Device("hip:0")
    assert d2.device_id == dev.device_id
    with pytest.raises(MorokHipError) as e:
        morok_amd.Device("HIP:99")
    assert e.value.code == 3


def test_lazy_allocation_and_roundtrip(dev):
    b = dev.buffer(4096)
    assert not b.is_allocated()
    with pytest.raises(MorokHipError) as e:
        b.raw_ptr_unallocated_ok()
    assert e.value.code == 4  # NotAllocated
    data = np.arange(1024, dtype=np.float32)
    b.copyin(data)
    assert b.is_allocated()
    assert np.array_equal(b.copyout(np.float32), data)


def test_copy_size_mismatch(dev):
    b = dev.buffer(64)
    with pytest.raises(MorokHipError) as e:
        b.copyin(np.zeros(15, np.float32))
    assert e.value.code == 1 and "expected 64, got 60" in e.value.message
    with pytest.raises(MorokHipError) as e:
        b.copyout(nbytes=32)
    assert e.value.code == 1
    other = dev.buffer(32)
    with pytest.raises(MorokHipError) as e:
        b.copy_from(other)
    assert e.value.code == 1


def test_views_share_id_and_memory(dev):
    base = dev.buffer(1024)
    base.copyin(np.arange(256, dtype=np.int32))
    v = base.view(256, 512)
    assert v.id == base.id and v.size == 512
    assert v.ptr == base.ptr + 256
    assert np.array_equal(v.copyout(np.int32), np.arange(64, 192, dtype=np.int32))
    v.copyin(np.full(128, -1, np.int32))
    out = base.copyout(np.int32)
    assert np.all(out[64:192] == -1) and out[63] == 63 and out[192] == 192
    vv = v.view(8, 16)
    assert vv.ptr == base.ptr + 264
    with pytest.raises(MorokHipError) as e:
        base.view(1000, 100)
    assert e.value.code == 6 and "exceeds buffer size 1024" in e.value.message


def test_copy_from_device_to_device(dev):
    a = morok_amd.Buffer.from_numpy(np.arange(100, dtype=np.float32), dev.device_id)
    b = dev.buffer(400)
    b.copy_from(a)
    assert np.array_equal(b.copyout(np.float32), np.arange(100, dtype=np.float32))


def test_lru_reuse_pointer_identity_and_zero_init(dev):
    dev.lru_clear()
    size = 123456
    p = dev.alloc(size)
    dev.free(p, size)
    assert dev.lru_cache_count(size) == 1
    assert dev.lru_cache_count(size, cpu_accessible=True) == 0  # key includes cpu_accessible
    q = dev.alloc(size)
    assert q == p and dev.lru_cache_count(size) == 0
    # dirty it, free, re-alloc with zero_init: same pointer, zeroed
    import ctypes as C

    junk = np.full(size, 0xAB, np.uint8)
    morok_amd._ffi.check(morok_amd.lib.mrk_hip_copyin(dev.device_id, q, 0, junk.ctypes.data_as(C.c_void_p), size))
    dev.free(q, size)
    r = dev.alloc(size, zero_init=True)
    assert r == p
    out = np.empty(size, np.uint8)
    morok_amd._ffi.check(morok_amd.lib.mrk_hip_copyout(dev.device_id, out.ctypes.data_as(C.c_void_p), r, 0, size))
    assert not out.any()
    dev.free(r, size)
    # at most 32 cached per key
    ptrs = [dev.alloc(4096) for _ in range(40)]
    for x in ptrs:
        dev.free(x, 4096)
    assert dev.lru_cache_count(4096) == 32
    dev.lru_clear()
    assert dev.lru_total_cached() == 0


def test_buffer_release_returns_to_lru(dev):
    dev.lru_clear()
    b = dev.buffer(7777).ensure_allocated()
    p = b.ptr
    v = b.view(0, 16)
    b.release()
    assert dev.lru_cache_count(7777) == 0  # a live view keeps the allocation
    v.release()
    assert dev.lru_cache_count(7777) == 1
    assert dev.buffer(7777).ptr == p


def test_managed_cpu_accessible_allocation(dev):
    b = dev.buffer(256, cpu_accessible=True)
    b.copyin(np.arange(64, dtype=np.int32))
    assert np.array_equal(b.copyout(np.int32), np.arange(64, dtype=np.int32))


def test_compile_load_execute_with_vars(dev):
    # the pattern of runtime/src/jit_loader.rs:795-871 (literal source, scalar args) on the GPU
    src = r"""
extern "C" __global__ void axpy(float* data0, const float* data1, const int n, const long long off) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) data0[i] = 2.0f * data1[i] + (float)off;
}"""
    spec = morok_amd.ProgramSpec.from_source("axpy", src, 2, ["n", "off"], [0, 1])
    prog = morok_amd.Program.create(morok_amd.compile_spec(spec), dev.device_id)
    assert prog.name == "axpy"
    n = 1000
    x = np.arange(n, dtype=np.float32)
    bx = morok_amd.Buffer.from_numpy(x, dev.device_id)
    by = dev.buffer(x.nbytes)
    prog.execute([by, bx], [n, 5_000_000_000 % 1000], (4, 1, 1), (256, 1, 1))
    assert np.array_equal(by.copyout(np.float32), 2 * x + 0)
    prog.execute([by, bx], [n, 7], (4, 1, 1), (256, 1, 1))
    assert np.array_equal(by.copyout(np.float32), 2 * x + 7)
    with pytest.raises(MorokHipError) as e:
        prog.execute([by], [n, 7], (4, 1, 1), (256, 1, 1))
    assert e.value.code == 11
    with pytest.raises(MorokHipError):
        prog.execute([by, bx], [n], (4, 1, 1), (256, 1, 1))
    with pytest.raises(MorokHipError):
        prog.execute([by, bx], [n, 7])  # no sizes recorded and none given
    with pytest.raises(MorokHipError):
        prog.execute([by, bx], [n, 7], (1, 1, 1), (2048, 1, 1))


def test_missing_entry_point(dev):
    spec = morok_amd.ProgramSpec.from_source("nope", 'extern "C" __global__ void other(float* a) { a[0] = 1; }', 1)
    with pytest.raises(MorokHipError) as e:
        morok_amd.Program.create(morok_amd.compile_spec(spec), dev.device_id)
    assert e.value.code == 8


def test_event_timing(dev):
    b = dev.buffer(1 << 20, zero_init=True).ensure_allocated()
    ms = morok_amd.time_launches(lambda: b.copy_from(b.view(0, 1 << 20)) if False else dev.synchronize(), 3, 1)
    assert ms >= 0.0
