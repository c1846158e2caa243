"""Parity of the fused HIP row softmax with the CPU oracle (3-kernel restatement of
Tensor::softmax) on identical seeded inputs.  Tolerance from the north star: <= 1e-5
relative for f32 elementwise results (each output is exp(x-m)/s, whose reductions are
held to 1e-4; the tighter bound is asserted)."""
import numpy as np
import pytest

import morok_amd
from morok_amd import ops, synth

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def _run(dev, x, variant=0, via_program=False):
    rows, cols = x.shape
    bx = morok_amd.Buffer.from_numpy(x, dev.device_id)
    by = dev.buffer(x.nbytes)
    if via_program:
        prog = morok_amd.Program.builtin("softmax_f32", [rows, cols], dev.device_id)
        prog.execute([by, bx])
    else:
        ops.softmax_f32(bx, by, rows, cols, dev.device_id, variant)
    return by.copyout(np.float32, (rows, cols))


def _check(y, ref, rtol=RTOL):
    assert np.all(np.isfinite(y))
    rel = np.abs(y - ref) / np.maximum(ref, np.float32(1e-30))
    # entries that underflow towards denormals carry no relative precision; bound them absolutely
    big = ref > 1e-30
    assert rel[big].max() <= rtol, rel[big].max()
    assert np.abs(y - ref).max() <= rtol * ref.max()


def _softmax_f64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


@pytest.mark.parametrize("shape", [(1, 4), (3, 8), (64, 256), (33, 1000), (17, 1024), (8, 2048), (5, 4100),
                                   (16, 8192), (7, 12), (4, 10000), (2, 8196), (9, 333)])
@pytest.mark.parametrize("variant", [0, 1])
def test_softmax_parity_shapes(dev, oracle, shape, variant):
    x = synth.normal(shape, 2, 0, sigma=2.0)
    _check(_run(dev, x, variant), oracle.softmax_f32(x))


@pytest.mark.parametrize("shape", [(64, 8191), (16, 12288), (8, 16384), (6, 32000), (5, 50257), (4, 65536),
                                   (3, 65537), (3, 131072), (2, 100003), (7, 8193)])
def test_softmax_long_and_unaligned_rows(dev, oracle, shape):
    """Rows beyond 8192 columns stay in registers up to 65536 (512 / 1024 work-items per row),
    longer ones take the two-sweep kernel; odd column counts give every row its own alignment."""
    x = synth.normal(shape, 2, 1, sigma=2.0)
    y = _run(dev, x)
    # The oracle adds a row's exponentials one after another in f32 like the CPU backend it
    # restates; over 10^5 terms that sum is itself 2.5e-5 off the exact one, so against the
    # oracle these rows are held to the 1e-4 of f32 reductions and to 1e-5 against float64.
    _check(y, oracle.softmax_f32(x), rtol=1e-4)
    _check(y, _softmax_f64(x), rtol=1e-5)


def test_softmax_rows_misaligned_differently_in_x_and_y(dev, oracle):
    """Views whose bases are not 16-byte aligned alike fall back to element-wise access."""
    rows, cols = 5, 70001
    x = synth.normal((rows, cols), 2, 2, sigma=2.0)
    bx = dev.buffer(x.nbytes + 64)
    by = dev.buffer(x.nbytes + 64)
    vx, vy = bx.view(4, x.nbytes), by.view(8, x.nbytes)
    vx.copyin(x)
    ops.softmax_f32(vx.ptr, vy.ptr, rows, cols, dev.device_id)
    y = vy.copyout(np.float32, (rows, cols))
    _check(y, oracle.softmax_f32(x), rtol=1e-4)
    _check(y, _softmax_f64(x), rtol=1e-5)


@pytest.mark.parametrize("shape", [(3, 8191), (5, 1001), (2, 70001), (4, 4096), (7, 33)])
def test_softmax_does_not_touch_neighbours(dev, oracle, shape):
    """NaNs right behind x in its allocation do not reach y, and nothing is written behind y."""
    rows, cols = shape
    x = synth.normal(shape, 2, 3, sigma=2.0)
    pad = np.full(1024, np.nan, np.float32)
    bx = morok_amd.Buffer.from_numpy(np.concatenate([x.reshape(-1), pad]), dev.device_id)
    by = morok_amd.Buffer.from_numpy(np.full(rows * cols + 1024, np.nan, np.float32), dev.device_id)
    ops.softmax_f32(bx, by, rows, cols, dev.device_id)
    out = by.copyout(np.float32)
    _check(out[: rows * cols].reshape(shape), oracle.softmax_f32(x), rtol=1e-4)
    assert np.all(np.isnan(out[rows * cols:]))


def test_softmax_config_slice_of_full_shape(dev, oracle):
    # rows of the benchmark shape [8192 x 8192], N(0, 2): a slice the oracle finishes quickly
    x = synth.normal((256, 8192), 2, 0, sigma=2.0)
    ref = oracle.softmax_f32(x)
    _check(_run(dev, x), ref)
    _check(_run(dev, x, via_program=True), ref)


def test_softmax_full_size_properties(dev):
    # full benchmark size: size-independent properties (row sums, range, shift invariance, argmax)
    rows = cols = 8192
    x = synth.normal((rows, cols), 2, 0, sigma=2.0)
    y = _run(dev, x)
    assert np.abs(y.sum(-1, dtype=np.float64) - 1.0).max() < 1e-4
    assert np.all(y > 0) and np.all(y <= 1)
    assert np.array_equal(y.argmax(-1), x.argmax(-1))
    y2 = _run(dev, x + np.float32(1.5))
    assert np.abs(y2 - y).max() <= 2e-6 * y.max() + 1e-9


def test_softmax_edge_values(dev):
    x = np.array([[1e4, -1e4, 1e4, 0.0], [-np.inf, 0.0, 0.0, -np.inf], [5.0, 5.0, 5.0, 5.0]], np.float32)
    y = _run(dev, x)
    assert np.allclose(y[0], [0.5, 0, 0.5, 0])
    assert np.allclose(y[1], [0, 0.5, 0.5, 0])
    assert np.allclose(y[2], 0.25)


def test_softmax_empty(dev):
    ops.softmax_f32(0, 0, 0, 128, dev.device_id)
    ops.softmax_f32(0, 0, 16, 0, dev.device_id)


@pytest.mark.parametrize("seed", range(24))
def test_softmax_random_shapes(dev, oracle, seed):
    rng = np.random.default_rng(4000 + seed)
    rows = int(rng.integers(1, 70))
    cols = int(rng.choice([rng.integers(1, 300), rng.integers(300, 9000), rng.integers(9000, 80000)]))
    x = synth.normal((rows, cols), 2, 50 + seed, sigma=float(rng.choice([0.5, 2.0, 8.0])))
    y = _run(dev, x, variant=int(seed & 1))
    _check(y, oracle.softmax_f32(x), rtol=1e-4)
    _check(y, _softmax_f64(x), rtol=1e-5)
