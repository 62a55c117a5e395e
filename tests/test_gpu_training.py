"""The whole training path in one loop on the GPU, in the shape of the reference's MNIST LUT-network sample
(samples/cpp/mnist/MnistDifferentiableLutSimple.cpp: DifferentiableLut6 layers with batch-norm in binary mode, a 6-to-1
reduction, softmax cross entropy, Adam), scaled down to a synthetic 10-class problem: every piece is parity-tested on its
own elsewhere; here they have to fit together (gradient signs, accumulation into dW, statistics hand-over, optimizer
tables) well enough to learn.  The first step is also checked against the same chain of CPU oracle calls."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32

I, O1, O2, CLASSES, N_AVG = 128, 384, 60, 10, 6
F = 512


def make_batch(rng, prototypes, frames, stride):
    label = rng.integers(0, CLASSES, frames)
    x = prototypes[label].T.copy()                                   # [I][frames] of 0 / 1
    flip = rng.random(x.shape) < 0.1
    x = np.where(flip, 1 - x, x).astype(F32)
    xs = np.zeros((I, stride), F32); xs[:, :frames] = x
    t = np.zeros((CLASSES, stride), F32); t[label, np.arange(frames)] = 1
    return xs, t


def test_lut_network_learns():
    import torch
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    rng = np.random.default_rng(2024)
    stride = synth.frame_stride_fp32(F)
    prototypes = rng.integers(0, 2, (CLASSES, I))
    idx1 = synth.wiring(rng, I, O1); idx2 = synth.wiring(rng, O1, O2)
    idx3 = np.arange(O2, dtype=np.int32).reshape(CLASSES, N_AVG)
    W1h = (0.5 + 0.01 * rng.standard_normal((O1, 64))).astype(F32)
    W2h = (0.5 + 0.01 * rng.standard_normal((O2, 64))).astype(F32)
    W1, W2 = dev(W1h), dev(W2h)
    dW1, dW2 = torch.zeros_like(W1), torch.zeros_like(W2)
    rm1, rv1 = torch.zeros(O1, device="cuda"), torch.ones(O1, device="cuda")
    rm2, rv2 = torch.zeros(O2, device="cuda"), torch.ones(O2, device="cuda")
    d_idx1, d_idx2, d_idx3 = dev(idx1), dev(idx2), dev(idx3)
    rev1, rev2 = ops.reverse_table(d_idx1, I), ops.reverse_table(d_idx2, O1)
    adam = ops.AdamState([W1, W2], [dW1, dW2], learning_rate=0.01)

    def forward(x, train):
        if train:
            y1, m1, r1 = ops.differentiable_lut_forward_training(6, x, d_idx1, W1, F, rm1, rv1)
            y2, m2, r2 = ops.differentiable_lut_forward_training(6, y1, d_idx2, W2, F, rm2, rv2)
        else:
            y1 = ops.differentiable_lut_forward_inference(6, x, d_idx1, W1, F, rm1, rv1); m1 = r1 = None
            y2 = ops.differentiable_lut_forward_inference(6, y1, d_idx2, W2, F, rm2, rv2); m2 = r2 = None
        y3 = ops.average_lut_forward(y2, d_idx3, F, False, False, mean=False)
        return y1, m1, r1, y2, m2, r2, y3

    losses, accuracies = [], []
    for step in range(120):
        xh, th = make_batch(rng, prototypes, F, stride)
        x, t = dev(xh), dev(th)
        ops.vector_clamp_(W1); ops.vector_clamp_(W2)
        y1, m1, r1, y2, m2, r2, y3 = forward(x, True)
        dy3, loss_buf, t_sum = ops.loss_softmax_cross_entropy(y3, t, CLASSES, 1, F)
        acc, cat = ops.metrics_categorical_accuracy(y3, t, CLASSES, 1, F)
        losses.append(-float(loss_buf.sum().item()) / t_sum)
        accuracies.append(int(acc.sum().item()) / int(cat.sum().item()))
        if step == 0:
            first = dict(x=xh, t=th, y3=host(y3), dy3=host(dy3), loss=losses[0], W1=host(W1), W2=host(W2))
        dW1.zero_(); dW2.zero_()
        dy2 = ops.average_lut_backward(dy3, d_idx3, O2, F)
        dy1 = ops.differentiable_lut_backward(6, y1, dy2, d_idx2, W2, dW2, F, m2, r2, rev2)
        ops.differentiable_lut_backward(6, x, dy1, d_idx1, W1, dW1, F, m1, r1, rev1)
        if step == 0:
            first.update(dW1=host(dW1), dW2=host(dW2))
        adam.step()

    print("loss %.3f -> %.3f, accuracy %.2f -> %.2f" % (losses[0], np.mean(losses[-10:]), accuracies[0], np.mean(accuracies[-10:])))
    # it learns: the loss falls well below log(10) and most of a fresh batch is classified, also through the inference path
    assert losses[0] > 2.0 and np.mean(losses[-10:]) < 0.3 * losses[0], (losses[0], losses[-10:])
    assert np.mean(accuracies[-10:]) > 0.9, accuracies[-10:]
    xh, th = make_batch(rng, prototypes, F, stride)
    y3 = forward(dev(xh), False)[-1]
    acc, cat = ops.metrics_categorical_accuracy(y3, dev(th), CLASSES, 1, F)
    assert int(acc.sum().item()) / int(cat.sum().item()) > 0.9

    # the first step against the same chain on the CPU oracle.  Forward: the chain as it ran (a binarized activation may differ
    # where its pre-activation sits within rounding of the threshold, and the next layer sees a whole step there).  Backward:
    # each layer on the oracle's own activations, statistics and incoming gradient, which keeps it at the single-layer tolerance.
    from test_gpu_chains_full_size import _backward_layer, _bn_output_fp64
    z, o = np.zeros(O1, F32), np.ones(O1, F32)
    y1r, m1r, r1r, _, _ = oracle.differentiable_lut_forward_training(6, first["x"], idx1, first["W1"], F, z, o)
    y2r, m2r, r2r, _, _ = oracle.differentiable_lut_forward_training(6, y1r, idx2, first["W2"], F, np.zeros(O2, F32), np.ones(O2, F32))
    y3r = oracle.average_lut_forward(y2r, idx3, F, False, False)
    assert np.mean(first["y3"][:, :F] != y3r[:, :F]) < 1e-3
    dy3r, lbr, tsr = oracle.loss_softmax_cross_entropy(y3r, first["t"], CLASSES, 1, F)
    assert abs(first["loss"] - (-lbr.sum() / tsr)) < 1e-3 * abs(first["loss"])
    dy2r = oracle.average_lut_backward(dy3r, idx3, O2, F)
    t2 = _bn_output_fp64(y1r, idx2, first["W2"], m2r, r2r, F)
    dy1r, _ = _backward_layer(ops, y1r, dy2r, idx2, first["W2"], F, m2r, r2r, t2, "second layer")        # dx, dW within 1e-4
    t1 = _bn_output_fp64(first["x"], idx1, first["W1"], m1r, r1r, F)
    _backward_layer(ops, first["x"], dy1r, idx1, first["W1"], F, m1r, r1r, t1, "first layer")
    # and the chain's own table gradients point the same way as the oracle chain's
    _, dW2r = oracle.differentiable_lut_backward(6, y1r, dy2r, idx2, first["W2"], F, m2r, r2r)
    cos = float((first["dW2"] * dW2r).sum() / (np.linalg.norm(first["dW2"]) * np.linalg.norm(dW2r)))
    assert cos > 0.999, cos
