"""The oracle's Reduce, LossMeanSquaredError and MetricsMeanSquaredError, pinned without a GPU: vectors written by the reference's own
host classes (tests/golden/reduce_mse.npz), the compiled reference where oracle/_ref is present, numpy in float64.
Reduce and the loss gradient are single fp32 operations per element in a fixed order: bit-exact.  The loss and the metric are sums of
doubles in the reference's order: equal to the last bit against the reference, 1e-12 relative against numpy."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reduce_mse.npz"))
F32 = np.float32


def mse_batches(y, t, F, batches, rsum):
    """the layer's bookkeeping around the oracle's per-batch loops -> (dy, loss, metric)"""
    nodes = y.shape[0]
    dy = np.zeros_like(y)
    loss = 0.0; acc = 0.0
    for b in range(batches):
        sl = slice(b * F, (b + 1) * F)
        d, loss = oracle.loss_mean_squared_error(np.ascontiguousarray(y[:, sl]), np.ascontiguousarray(t[:, sl]), F, reduction_sum=rsum, loss=loss)
        dy[:, sl] = d
        acc = oracle.metrics_mean_squared_error(np.ascontiguousarray(y[:, sl]), np.ascontiguousarray(t[:, sl]), F, accuracy=acc)
    frames = F * batches
    return dy, (loss if rsum else loss / frames), acc / frames


def test_reference_vectors():
    for k in range(int(GOLD["reduce_count"][0])):
        p = "r%d_" % k
        I, O, F, integ = [int(v) for v in GOLD[p + "geom"]]
        assert np.array_equal(oracle.reduce_forward(GOLD[p + "x"], O, F), GOLD[p + "y"]), k
        assert np.array_equal(oracle.reduce_backward(GOLD[p + "dy"], I, F), GOLD[p + "dx"]), k
        assert np.array_equal(oracle.bit_reduce_forward(GOLD[p + "xbits"], O, F, F), GOLD[p + "y_from_bits"]), k
    for k in range(int(GOLD["mse_count"][0])):
        p = "e%d_" % k
        nodes, F, batches, rsum = [int(v) for v in GOLD[p + "geom"]]
        dy, loss, metric = mse_batches(GOLD[p + "y"], GOLD[p + "t"], F, batches, bool(rsum))
        assert np.array_equal(dy, GOLD[p + "dy"]), k
        assert loss == GOLD[p + "loss_metric"][0] and metric == GOLD[p + "loss_metric"][1], k


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_against_compiled_reference():
    rng = np.random.default_rng(41)
    for (I, O, F) in [(60, 12, 77), (9, 9, 3), (128, 2, 200)]:
        x = rng.standard_normal((I, F)).astype(F32); dy = rng.standard_normal((O, F)).astype(F32)
        y, dx, _ = oracle.ref_reduce(x, O, F, dy=dy)
        assert np.array_equal(oracle.reduce_forward(x, O, F), y) and np.array_equal(oracle.reduce_backward(dy, I, F), dx)
        xb = synth.bernoulli_bits(rng, I, F)
        yb, _, _ = oracle.ref_reduce(xb, O, F, bit=True)
        assert np.array_equal(oracle.bit_reduce_forward(xb, O, F, F), yb)
    for (nodes, F, batches, rsum) in [(7, 50, 2, False), (20, 9, 1, True), (4, 300, 3, False)]:
        y = rng.random((nodes, F * batches)).astype(F32); t = rng.random((nodes, F * batches)).astype(F32)
        want = oracle.ref_mean_squared_error(y, t, F, batches, rsum)
        got = mse_batches(y, t, F, batches, rsum)
        assert np.array_equal(got[0], want[0]) and got[1] == want[1] and got[2] == want[2]


def test_numpy_means():
    rng = np.random.default_rng(42)
    I, O, F = 48, 6, 90
    x = rng.standard_normal((I, F)).astype(F32)
    y = oracle.reduce_forward(x, O, F)
    assert np.abs(y - x.astype(np.float64).reshape(I // O, O, F).mean(axis=0)).max() < 1e-6
    dy = rng.standard_normal((O, F)).astype(F32)
    dx = oracle.reduce_backward(dy, I, F)
    assert np.array_equal(dx, np.tile(dy / F32(I // O), (I // O, 1)))
    xb = synth.bernoulli_bits(rng, I, F)
    b = synth.unpack_bits(xb, F).astype(np.float64) * 2 - 1
    assert np.abs(oracle.bit_reduce_forward(xb, O, F, F) - b.reshape(I // O, O, F).mean(axis=0)).max() < 1e-6
    # a layer with as many outputs as inputs is the identity
    assert np.array_equal(oracle.reduce_forward(x, I, F), x)
    nodes, F = 9, 120
    y = rng.random((nodes, F)).astype(F32); t = rng.random((nodes, F)).astype(F32)
    dy, loss, metric = mse_batches(y, t, F, 1, False)
    d = y.astype(np.float64) - t
    assert abs(loss - (d * d).mean()) < 1e-7 and abs(metric - (d * d).mean()) < 1e-7
    assert np.abs(dy - 2 * d / (nodes * F)).max() < 1e-9
    _, loss_sum, _ = mse_batches(y, t, F, 1, True)
    assert abs(loss_sum - (d * d).sum()) < 1e-4
    # a NaN in the output poisons its own gradient and is left out of the loss
    y2 = y.copy(); y2[3, 7] = np.nan
    dy2, loss2, _ = mse_batches(y2, t, F, 1, False)
    assert np.isnan(dy2[3, 7]) and np.isfinite(loss2) and abs(loss2 - ((d * d).sum() - d[3, 7] ** 2) / (nodes * F)) < 1e-7
