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


def _check(y, ref):
    assert np.all(np.isfinite(y))
    rel = np.abs(y - ref) / np.maximum(ref, np.float32(1e-30))
    # entries that underflow towards denormals carry no relative precision; bound them absolutely
    big = ref > 1e-30
    assert rel[big].max() <= RTOL, rel[big].max()
    assert np.abs(y - ref).max() <= RTOL * ref.max()


@pytest.mark.parametrize("shape", [(1, 4), (3, 8), (64, 256), (33, 1000), (17, 1024), (8, 2048), (5, 4100),
                                   (16, 8192), (7, 12), (4, 10000), (2, 8196), (9, 333)])
@pytest.mark.parametrize("variant", [0, 1])
def test_softmax_parity_shapes(dev, oracle, shape, variant):
    x = synth.normal(shape, 2, 0, sigma=2.0)
    _check(_run(dev, x, variant), oracle.softmax_f32(x))


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
