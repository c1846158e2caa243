"""Deterministic synthetic inputs (the reference has no RNG: tensor/src/nn/mod.rs:304).

Counter-based generator: value i of tensor `tensor_id` under `seed` is a pure function of
(seed, tensor_id, i) through SplitMix64, so any slice can be generated independently and
the same bytes are fed to the CPU oracle and to the HIP path.  Normals use Box-Muller in
float64 and are then rounded to the requested dtype.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _splitmix64(x):
    x = (x + _GOLDEN).astype(np.uint64)
    z = x
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _bits(seed, tensor_id, n, stream=0, start=0):
    with np.errstate(over="ignore"):
        key = _splitmix64(np.array([seed * 0x1000003 + tensor_id * 0x10001 + stream], dtype=np.uint64))[0]
        idx = np.arange(start, start + n, dtype=np.uint64)
        return _splitmix64(idx * np.uint64(0xD6E8FEB86659FD93) + key)


def _unit(seed, tensor_id, n, stream=0, start=0):
    """Uniform float64 in (0, 1)."""
    b = _bits(seed, tensor_id, n, stream, start)
    return ((b >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def uniform(shape, seed, tensor_id=0, lo=-1.0, hi=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=dtype)
    step = 1 << 22
    for s in range(0, n, step):
        m = min(step, n - s)
        out[s:s + m] = (lo + (hi - lo) * _unit(seed, tensor_id, m, 0, s)).astype(dtype)
    return out.reshape(shape)


def normal(shape, seed, tensor_id=0, sigma=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=dtype)
    step = 1 << 22
    for s in range(0, n, step):
        m = min(step, n - s)
        u1 = _unit(seed, tensor_id, m, 1, s)
        u2 = _unit(seed, tensor_id, m, 2, s)
        out[s:s + m] = (sigma * np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(dtype)
    return out.reshape(shape)


def randint(shape, seed, tensor_id=0, high=2, dtype=np.int32):
    n = int(np.prod(shape))
    return (_bits(seed, tensor_id, n, 3) % np.uint64(high)).astype(dtype).reshape(shape)


def to_bf16(x):
    """float32 array -> uint16 array of bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def from_bf16(b):
    """uint16 bfloat16 bit patterns -> float32."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def normal_bf16(shape, seed, tensor_id=0, sigma=1.0):
    return to_bf16(normal(shape, seed, tensor_id, sigma))
