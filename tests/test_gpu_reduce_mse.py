"""GPU parity of Reduce, LossMeanSquaredError and MetricsMeanSquaredError (through the C ABI) against the CPU oracle and against the
vectors that the reference's own host classes wrote (tests/golden/reduce_mse.npz).  Reduce and the loss gradient are bit-exact.  The
loss and the metric are sums of doubles taken in another order than the host's single running sum: 1e-12 relative."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reduce_mse.npz"))
SUM_RTOL = 1e-12


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


@pytest.mark.parametrize("shape", [(70, 10, 1024), (70, 10, 37), (12, 12, 5), (96, 3, 130), (6144, 1024, 300), (4096, 2, 64), (3, 1, 1)])
def test_reduce(ops, shape):
    I, O, F = shape
    rng = np.random.default_rng(sum(shape))
    stride = synth.frame_stride_fp32(F)
    x = _pad(rng.standard_normal((I, F)).astype(F32), stride)
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    y = host(ops.reduce_forward(dev(x), O, F))
    assert np.array_equal(y[:, :F], oracle.reduce_forward(x, O, F)[:, :F])
    dx = host(ops.reduce_backward(dev(dy), I, F))
    assert np.array_equal(dx[:, :F], oracle.reduce_backward(dy, I, F)[:, :F])
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
    yb = host(ops.bit_reduce_forward(dev(xb), O, F, stride))
    assert np.array_equal(yb[:, :F], oracle.bit_reduce_forward(xb, O, F, stride)[:, :F])


def run_mse(ops, y, t, F, batches, rsum, buf_size=1024):
    import torch
    nodes = y.shape[0]
    stride = synth.frame_stride_fp32(F)
    loss_buf = torch.zeros(buf_size, dtype=torch.float64, device="cuda")
    acc_buf = torch.zeros(buf_size, dtype=torch.float64, device="cuda")
    dy = np.zeros_like(y)
    for b in range(batches):
        sl = slice(b * F, (b + 1) * F)
        yd = dev(_pad(np.ascontiguousarray(y[:, sl]), stride)); td = dev(_pad(np.ascontiguousarray(t[:, sl]), stride))
        dy[:, sl] = host(ops.loss_mean_squared_error(yd, td, F, loss_buf, reduction_sum=rsum))[:, :F]
        ops.metrics_mean_squared_error(yd, td, F, acc_buf)
    frames = F * batches
    loss = float(host(loss_buf).sum())
    return dy, (loss if rsum else loss / frames), float(host(acc_buf).sum()) / frames


def test_reference_vectors(ops):
    for k in range(int(GOLD["reduce_count"][0])):
        p = "r%d_" % k
        I, O, F, integ = [int(v) for v in GOLD[p + "geom"]]
        stride = synth.frame_stride_fp32(F)
        assert np.array_equal(host(ops.reduce_forward(dev(_pad(GOLD[p + "x"], stride)), O, F))[:, :F], GOLD[p + "y"]), k
        assert np.array_equal(host(ops.reduce_backward(dev(_pad(GOLD[p + "dy"], stride)), I, F))[:, :F], GOLD[p + "dx"]), k
        xb = _pad(GOLD[p + "xbits"], synth.frame_stride_bit(F))
        assert np.array_equal(host(ops.bit_reduce_forward(dev(xb), O, F, stride))[:, :F], GOLD[p + "y_from_bits"]), k
    for k in range(int(GOLD["mse_count"][0])):
        p = "e%d_" % k
        nodes, F, batches, rsum = [int(v) for v in GOLD[p + "geom"]]
        dy, loss, metric = run_mse(ops, GOLD[p + "y"], GOLD[p + "t"], F, batches, bool(rsum))
        assert np.array_equal(dy, GOLD[p + "dy"]), k
        want_loss, want_metric = GOLD[p + "loss_metric"]
        assert abs(loss - want_loss) <= SUM_RTOL * abs(want_loss) and abs(metric - want_metric) <= SUM_RTOL * abs(want_metric), k


@pytest.mark.parametrize("shape", [(10, 1024, 1), (784, 300, 2), (1, 5, 1), (130, 2500, 1), (65, 64, 3)])
def test_mean_squared_error(ops, shape):
    nodes, F, batches = shape
    rng = np.random.default_rng(sum(shape))
    y = rng.random((nodes, F * batches)).astype(F32); t = (rng.random((nodes, F * batches)) > 0.5).astype(F32)
    for rsum in (False, True):
        for buf_size in (1024, 7, 1):
            dy, loss, metric = run_mse(ops, y, t, F, batches, rsum, buf_size)
            acc_l = 0.0; acc_m = 0.0
            for b in range(batches):
                sl = slice(b * F, (b + 1) * F)
                d, acc_l = oracle.loss_mean_squared_error(np.ascontiguousarray(y[:, sl]), np.ascontiguousarray(t[:, sl]), F, reduction_sum=rsum, loss=acc_l)
                assert np.array_equal(dy[:, sl], d), (rsum, buf_size, b)
                acc_m = oracle.metrics_mean_squared_error(np.ascontiguousarray(y[:, sl]), np.ascontiguousarray(t[:, sl]), F, accuracy=acc_m)
            want_loss = acc_l if rsum else acc_l / (F * batches)
            assert abs(loss - want_loss) <= SUM_RTOL * abs(want_loss), (rsum, buf_size)
            assert abs(metric - acc_m / (F * batches)) <= SUM_RTOL * abs(acc_m / (F * batches)), (rsum, buf_size)


def test_a_nan_output_is_left_out_of_the_loss(ops):
    import torch
    rng = np.random.default_rng(5)
    nodes, F = 9, 120
    stride = synth.frame_stride_fp32(F)
    y = rng.random((nodes, F)).astype(F32); t = rng.random((nodes, F)).astype(F32)
    y[3, 7] = np.nan
    buf = torch.zeros(1024, dtype=torch.float64, device="cuda")
    dy = host(ops.loss_mean_squared_error(dev(_pad(y, stride)), dev(_pad(t, stride)), F, buf))
    d, want = oracle.loss_mean_squared_error(y, t, F)
    assert np.isnan(dy[3, 7]) and np.array_equal(np.nan_to_num(dy[:, :F], nan=7.0), np.nan_to_num(d, nan=7.0))
    got = float(host(buf).sum())
    assert np.isfinite(got) and abs(got - want) <= SUM_RTOL * abs(want)


def test_rejected_arguments(ops):
    import torch
    from binarybrain_amd import capi
    x = torch.zeros((10, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.BbhipError):
        ops.reduce_forward(x, 3, 64)                    # 10 inputs do not fold into 3 outputs
    with pytest.raises(capi.BbhipError):
        ops.reduce_forward(x, 5, 65)
    with pytest.raises(capi.BbhipError):
        ops.reduce_backward(torch.zeros((3, 64), dtype=torch.float32, device="cuda"), 10, 64)
    with pytest.raises(capi.BbhipError):
        ops.loss_mean_squared_error(x, x.clone(), 65, torch.zeros(8, dtype=torch.float64, device="cuda"))
