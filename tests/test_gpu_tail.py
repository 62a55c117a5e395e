"""GPU parity of AverageLut, LossSoftmaxCrossEntropy and MetricsCategoricalAccuracy (through the C ABI) against the CPU
oracle.  AverageLut and the accuracy counts are sums in a fixed order, votes and integers: bit-exact.  The loss goes
through exp and log, whose device and host library versions may differ in the last place: tolerances are written at
the assertions."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "tail.npz"))
LOSS_RTOL = 1e-5      # batch loss, relative
DY_ATOL = 2e-6        # dy * t_sum / t_max (softmax minus target, values in [-1, 1]), absolute


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


AVERAGE_SHAPES = [
    # n, I, O, frames
    (7, 70, 10, 1024),          # the tail of the MNIST classifier
    (7, 70, 10, 37),
    (4, 9, 5, 64),
    (1, 3, 3, 5),
    (8, 8, 2, 100),
    (15, 200, 33, 300),
    (16, 64, 7, 257),
    (300, 40, 3, 70),           # more inputs than the bit-plane counter covers
    (6, 6144, 1024, 130),
]


@pytest.mark.parametrize("shape", AVERAGE_SHAPES)
def test_average_lut(ops, shape):
    n, I, O, F = shape
    rng = np.random.default_rng(sum(shape))
    idx = rng.integers(0, I, (O, n)).astype(np.int32)
    stride = synth.frame_stride_fp32(F)
    x = _pad((rng.random((I, F)) * 2 - 1).astype(F32), stride)
    x[rng.random(x.shape) < 0.05] = 0.0
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    for bin_in in (False, True):
        for bin_out in (False, True):
            for mean in (False, True):
                y = host(ops.average_lut_forward(dev(x), dev(idx), F, bin_in, bin_out, mean=mean))
                assert np.array_equal(y[:, :F], oracle.average_lut_forward(x, idx, F, bin_in, bin_out, mean=mean)[:, :F]), (bin_in, bin_out, mean)
    dx = host(ops.average_lut_backward(dev(dy), dev(idx), I, F))
    assert np.array_equal(dx, oracle.average_lut_backward(dy, idx, I, F))          # padding columns included: zero
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
    yb = host(ops.bit_average_lut_forward(dev(xb), dev(idx), F))
    assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(oracle.bit_average_lut_forward(xb, idx, F), F))


def test_average_lut_reference_vectors(ops):
    for k in range(int(GOLD["average_count"][0])):
        n, I, O, F, bin_in, bin_out = [int(v) for v in GOLD["a%d_geom" % k]]; q = "a%d_" % k
        idx = GOLD[q + "idx"]
        y = host(ops.average_lut_forward(dev(GOLD[q + "x"]), dev(idx), F, bool(bin_in), bool(bin_out), mean=False))      # vectors of the host loop
        assert np.array_equal(y, GOLD[q + "y"]), k
        dx = host(ops.average_lut_backward(dev(GOLD[q + "dy"]), dev(idx), I, F))
        assert np.array_equal(dx, GOLD[q + "dx"]), k
        yb = host(ops.bit_average_lut_forward(dev(GOLD[q + "xbits"]), dev(idx), F))
        assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(GOLD[q + "ybits"], F)), k


def test_average_lut_serial_wiring_and_unused_inputs(ops):
    # inputs [o*n, (o+1)*n) feed node o; the inputs after the last node feed nothing and receive a zero gradient
    n, O, F = 7, 10, 200
    I = n * O + 5
    idx = np.arange(n * O, dtype=np.int32).reshape(O, n)
    rng = np.random.default_rng(3)
    stride = synth.frame_stride_fp32(F)
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    dx = host(ops.average_lut_backward(dev(dy), dev(idx), I, F))
    assert np.array_equal(dx[:n * O, :F], np.repeat(dy[:, :F] / F32(n), n, axis=0))
    assert not dx[n * O:].any() and not dx[:, F:].any()


def _targets(rng, ch, pix, F, weighted=False):
    t = np.zeros((ch * pix, F), F32)
    for f in range(F):
        for p in range(pix):
            if weighted and rng.random() < 0.3:
                continue
            t[int(rng.integers(0, ch)) * pix + p, f] = F32(rng.integers(1, 4) * 0.5) if weighted else 1.0
    return t


def _check_loss(ops, y, t, ch, pix, F, stride):
    ys, ts = _pad(y, stride), _pad(t, stride)
    dy_ref, lb_ref, t_sum = oracle.loss_softmax_cross_entropy(ys, ts, ch, pix, F)
    dy, lb, t_sum_dev = ops.loss_softmax_cross_entropy(dev(ys), dev(ts), ch, pix, F)
    assert t_sum_dev == t_sum
    dy, lb = host(dy), host(lb)
    t_max = max(float(t.reshape(ch, pix, F).sum(axis=0).max()), 1e-30)
    assert np.abs(dy[:, :F] - dy_ref[:, :F]).max() * t_sum / t_max <= DY_ATOL
    loss, loss_ref = -lb.sum() / t_sum, -lb_ref.sum() / t_sum
    assert abs(loss - loss_ref) <= LOSS_RTOL * abs(loss_ref)
    assert np.allclose(lb, lb_ref, rtol=LOSS_RTOL, atol=1e-6 * t_max)
    acc, cat = ops.metrics_categorical_accuracy(dev(ys), dev(ts), ch, pix, F)
    acc_ref, cat_ref = oracle.metrics_categorical_accuracy(ys, ts, ch, pix, F)
    assert np.array_equal(host(acc), acc_ref) and np.array_equal(host(cat), cat_ref)
    return loss, dy


@pytest.mark.parametrize("shape", [(10, 1, 1024), (10, 1, 33), (4, 6, 17), (3, 5, 300), (2, 1, 1), (21, 64, 70), (1000, 1, 65)])
@pytest.mark.parametrize("kind", ["onehot", "sharp", "weighted", "ties"])
def test_loss_and_accuracy(ops, shape, kind):
    ch, pix, F = shape
    rng = np.random.default_rng(ch * 1000 + pix * 10 + F)
    y = (rng.standard_normal((ch * pix, F)) * (30.0 if kind == "sharp" else 1.0)).astype(F32)
    if kind == "ties":
        y = np.round(y)
    t = _targets(rng, ch, pix, F, weighted=(kind == "weighted"))
    if not t.any():
        t[0, 0] = 1
    _check_loss(ops, y, t, ch, pix, F, synth.frame_stride_fp32(F))


def test_loss_known_answers_of_the_reference_test(ops):
    # tests/gtest/LossSoftmaxCrossEntropyTest.cpp:8-92: NumPy goldens, loss within 1e-4, dy within 1e-6
    from test_oracle_tail import DX_TABLE, KNOWN_LOSS, known_answer_buffers
    y, t = known_answer_buffers()
    loss, dy = _check_loss(ops, y, t, 10, 1, 5, synth.frame_stride_fp32(5))
    assert abs(loss - KNOWN_LOSS) < 1e-4
    assert np.abs(dy[:, :5].T - DX_TABLE).max() < 1e-6


def test_loss_and_accuracy_reference_vectors(ops):
    for k in range(int(GOLD["loss_count"][0])):
        ch, pix, F = [int(v) for v in GOLD["l%d_geom" % k]]; q = "l%d_" % k
        loss, dy = _check_loss(ops, GOLD[q + "y"], GOLD[q + "t"], ch, pix, F, synth.frame_stride_fp32(F))
        assert abs(loss - GOLD[q + "loss"][0]) <= LOSS_RTOL * abs(GOLD[q + "loss"][0])
        t_sum = float(GOLD[q + "t"].sum(dtype=np.float64))
        t_max = float(GOLD[q + "t"].reshape(ch, pix, F).sum(axis=0).max())
        assert np.abs(dy[:, :F] - GOLD[q + "dy"]).max() * t_sum / t_max <= DY_ATOL
        acc, cat = ops.metrics_categorical_accuracy(dev(GOLD[q + "y"]), dev(GOLD[q + "t"]), ch, pix, F)
        assert int(host(acc).sum()) / int(host(cat).sum()) == GOLD[q + "metric"][0]


def test_loss_size_independent_properties(ops):
    # a batch as large as the benchmark's frames: one-hot dy sums to zero per pixel, equal logits give log(ch)
    ch, pix, F = 10, 1, 8192
    rng = np.random.default_rng(11)
    stride = synth.frame_stride_fp32(F)
    t = _pad(_targets(rng, ch, pix, F), stride)
    y = _pad(rng.standard_normal((ch, F)).astype(F32), stride)
    dy, lb, t_sum = ops.loss_softmax_cross_entropy(dev(y), dev(t), ch, pix, F)
    assert t_sum == F
    assert np.abs(host(dy)[:, :F].astype(np.float64).sum(axis=0)).max() * t_sum < 1e-6
    dy0, lb0, _ = ops.loss_softmax_cross_entropy(dev(np.zeros_like(y)), dev(t), ch, pix, F)
    assert abs(-host(lb0).sum() / t_sum - np.log(ch)) < 1e-5
    acc, cat = ops.metrics_categorical_accuracy(dev(t), dev(t), ch, pix, F)
    assert int(host(acc).sum()) == F and int(host(cat).sum()) == F


def test_rejected_arguments(ops):
    import torch
    x = torch.zeros((4, 64), device="cuda"); idx = torch.zeros((2, 3), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError):
        ops.average_lut_forward(x, idx, 0)                       # no frames
    with pytest.raises(RuntimeError):
        ops.average_lut_forward(x, idx, 65)                      # frames beyond the row pitch
    with pytest.raises(RuntimeError):
        ops.average_lut_backward(x[:2], idx, 0, 64)              # no input nodes
    with pytest.raises(RuntimeError):
        ops.loss_softmax_cross_entropy(x, x, 4, 1, 100, t_sum=1.0)
    with pytest.raises(RuntimeError):
        ops.metrics_categorical_accuracy(x, x, 4, 1, 0)


def test_average_lut_both_conventions(ops):
    """bbhip_fp32_AverageLut_Forward follows the reference's CUDA kernel of that name, sum * (1 / n), bit for bit;
    bbhip_fp32_AverageLut_ForwardSum its host loop, the plain sum; binarized outputs are the same in both, and so is the
    backward pass (dy / n)."""
    rng = np.random.default_rng(77)
    for n in (6, 7, 8):
        I, O, F = 90, 15, 333
        S = synth.frame_stride_fp32(F)
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        x = np.zeros((I, S), np.float32); x[:, :F] = rng.standard_normal((I, F))
        y = host(ops.average_lut_forward(dev(x), dev(idx), F, False, False))             # the entry's own convention: the mean
        ys = host(ops.average_lut_forward(dev(x), dev(idx), F, False, False, mean=False))
        yb = host(ops.average_lut_forward(dev(x), dev(idx), F, True, True))
        ybs = host(ops.average_lut_forward(dev(x), dev(idx), F, True, True, mean=False))
        assert np.array_equal(y[:, :F], oracle.average_lut_forward(x, idx, F, False, False, mean=True)[:, :F])
        assert np.array_equal(ys[:, :F], oracle.average_lut_forward(x, idx, F, False, False)[:, :F])
        assert np.array_equal(yb[:, :F], oracle.average_lut_forward(x, idx, F, True, True)[:, :F])
        assert np.array_equal(yb[:, :F], ybs[:, :F])
        # the two differ by exactly the fp32 reciprocal of n
        assert np.array_equal(y[:, :F], (ys[:, :F] * (np.float32(1.0) / np.float32(n))).astype(np.float32))


@pytest.mark.parametrize("case", [(70, 10, 7, 1024, False), (70, 10, 7, 1000, True), (30, 5, 3, 5000, False), (176, 16, 9, 37, False), (12, 2, 6, 64, True)])
@pytest.mark.parametrize("mean", [True, False])
def test_classifier_tail_in_one_launch(ops, case, mean):
    """bbhip_fp32_ClassifierTail_ForwardBackward = AverageLut forward + softmax cross entropy + accuracy + AverageLut backward: every output
    equals, bit for bit, what the four entries give called one after the other (and those are checked against the oracle above)."""
    import torch
    I, CH, n, F, bin_in = case
    rng = np.random.default_rng(I + CH + n + F)
    S = synth.frame_stride_fp32(F)
    idx = rng.integers(0, I - 2, (CH, n)).astype(np.int32)               # the last two inputs feed no node: their gradient is 0
    if I == 70:
        idx = np.arange(70, dtype=np.int32).reshape(10, 7)               # the classifier's own wiring
    x = np.zeros((I, S), np.float32); x[:, :F] = rng.integers(0, 2, (I, F)) if I == 70 else rng.standard_normal((I, F))
    t = np.zeros((CH, S), np.float32)
    label = rng.integers(0, CH, F)
    t[label, np.arange(F)] = 1.0
    t[:, F // 2] = 0.0                                                   # a frame without a target: not counted by the accuracy
    xd, td, idxd = dev(x), dev(t), dev(idx)
    y0 = ops.average_lut_forward(xd, idxd, F, bin_in, False, mean=mean)
    dy0, loss0, t_sum = ops.loss_softmax_cross_entropy(y0, td, CH, 1, F)
    acc0, cat0 = ops.metrics_categorical_accuracy(y0, td, CH, 1, F)
    dx0 = ops.average_lut_backward(dy0, idxd, I, F)
    y1, dx1, loss1, acc1, cat1, dy1 = ops.classifier_tail(xd, idxd, td, F, t_sum=t_sum, binarize_input=bin_in, mean=mean, want_dy=True)
    assert torch.equal(y0[:, :F], y1[:, :F]) and torch.equal(dy0[:, :F], dy1[:, :F])
    assert torch.equal(loss0, loss1) and torch.equal(acc0, acc1) and torch.equal(cat0, cat1)
    assert torch.equal(dx0, dx1)                                         # whole rows: the columns past the last frame are 0 in both
    assert I == 70 or not host(dx1)[I - 2:].any()
    # the outputs that the caller does not want may be left out
    _, dx2, loss2, acc2, _, _ = ops.classifier_tail(xd, idxd, td, F, t_sum=t_sum, binarize_input=bin_in, mean=mean, want_y=False, want_accuracy=False)
    assert torch.equal(dx0, dx2) and torch.equal(loss0, loss2) and acc2 is None


def test_classifier_tail_limits(ops):
    import torch
    x = torch.zeros((300, 64), device="cuda"); t = torch.zeros((4, 64), device="cuda")
    with pytest.raises(RuntimeError):
        ops.classifier_tail(x, torch.zeros((4, 3), dtype=torch.int32, device="cuda"), t, 64, t_sum=1.0)          # too many input nodes for one launch
    with pytest.raises(RuntimeError):
        ops.classifier_tail(x[:20], torch.zeros((17, 3), dtype=torch.int32, device="cuda"), torch.zeros((17, 64), device="cuda"), 64, t_sum=1.0)
