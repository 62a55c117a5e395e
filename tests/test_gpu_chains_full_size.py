"""The two multi-layer configurations at their full sizes, as chains: the classifier training step (DifferentiableLut6
784 -> 6144 -> 1024 -> 70 with batch-norm in binary mode, AverageLut 7 -> 1, softmax cross entropy, accuracy, Adam; 1024
frames) and the convolutional block (256 images of 3 x 32 x 32: Im2Col 3 x 3 -> DifferentiableLut6 27 -> 216 -> 36 per pixel ->
Col2Im -> StochasticMaxPooling2x2, forward and backward).

A chain of binarizing layers amplifies last-bit differences: one activation that lands on the other side of 0.5 changes the
next layer's input by a whole step.  To keep every layer at the tolerances of the single-layer tests (forward exact except
frames whose fp64 pre-activation lies within 2e-6 of the threshold; dW and dx within 1e-4), each device layer is fed the
ORACLE's activations and gradients of the layer before it, so what is compared is always one layer's work on identical
inputs, at the real shapes and row pitches.  The same holds for the hard-tanh window of the backward pass: where the fp64
batch-norm output of a (node, frame) pair lies within 1e-5 of an edge of the window, whether the gradient passes is a matter
of the last bit, and dy is zeroed for those pairs on both sides."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import assert_bwd, dev, host, rel_err

pytestmark = pytest.mark.gpu
F32 = np.float32
GAMMA, BETA, BIAS = 0.3, 0.5, 0.25


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


def _bn_output_fp64(x, idx, W, mean, rstd, F, gamma=GAMMA, beta=BETA):
    """fp64 batch-norm output t [O, F] of a binary-mode DifferentiableLut6 layer: with inputs mapped to 0.25 / 0.75 the LUT
    output of a frame is one of the 64 values V[o][corner], V = W K with K[i][c] = prod_j (bit_j(i) ? x_j(c) : 1 - x_j(c))."""
    lo, hi = 0.5 - BIAS, 0.5 + BIAS
    K = np.ones((64, 64))
    for i in range(64):
        for c in range(64):
            for j in range(6):
                xv = hi if (c >> j) & 1 else lo
                K[i, c] *= xv if (i >> j) & 1 else 1.0 - xv
    V = W.astype(np.float64) @ K                                             # [O, 64]
    bits = (x[:, :F] > 0.5)
    corner = np.zeros((idx.shape[0], F), np.int64)
    for j in range(6):
        corner |= bits[idx[:, j]].astype(np.int64) << j
    v = np.take_along_axis(V, corner, axis=1)
    return ((v - mean.astype(np.float64)[:, None]) * rstd.astype(np.float64)[:, None]) * gamma + beta


def _forward_layer(ops, x_ref, idx, W, F, stride, what):
    """one training forward on the oracle's input: statistics, then the binarized output exact away from the threshold"""
    import torch
    O = idx.shape[0]
    y_ref, mean_ref, rstd_ref, _, _ = oracle.differentiable_lut_forward_training(6, x_ref, idx, W, F, np.zeros(O, F32), np.ones(O, F32))
    y, mean, rstd = ops.differentiable_lut_forward_training(6, dev(x_ref), dev(idx), dev(W), F, torch.zeros(O, device="cuda"),
                                                            torch.ones(O, device="cuda"))
    assert rel_err(host(mean), mean_ref) <= 1e-5, what
    # 1 / sqrt(variance): the oracle forms E[y^2] - E[y]^2 in fp32 as the reference does and loses digits where the variance is
    # small (binarized inputs and tables near 0.5 give variances of a few 1e-4); a float64 evaluation arbitrates
    lut64 = _bn_output_fp64(x_ref, idx, W, np.zeros(O, F32), np.ones(O, F32), F, gamma=1.0, beta=0.0)
    rstd64 = 1.0 / np.sqrt(np.maximum(1e-5, lut64.var(axis=1)))
    assert np.abs(host(rstd) / rstd64 - 1.0).max() <= 1e-4 and np.abs(rstd_ref / rstd64 - 1.0).max() <= 2e-3, what
    t64 = _bn_output_fp64(x_ref, idx, W, mean_ref, rstd_ref, F)
    diff = host(y)[:, :F] != y_ref[:, :F]
    assert not (diff & (np.abs(t64 - 0.5) >= 2e-6)).any(), "%s: activations differ away from the threshold" % what
    assert diff.mean() <= 1e-4, what
    return y_ref, mean_ref, rstd_ref, t64


def _backward_layer(ops, x_ref, dy_ref, idx, W, F, mean_ref, rstd_ref, t64, what, nodes=None):
    """one backward on the oracle's input, statistics and incoming gradient (zeroed where the hard-tanh window is decided by the
    last bit); returns the oracle's dx and dW for the layer before.  nodes: the oracle (single-threaded, as the reference's
    backward) checks this slice of the nodes as a layer of its own, the device runs the whole layer and the slice."""
    import torch
    I, O = x_ref.shape[0], idx.shape[0]
    near = (np.abs(t64) < 1e-5) | (np.abs(t64 - 1.0) < 1e-5)
    assert near.mean() <= 1e-3
    dy_ref = dy_ref.copy()
    dy_ref[:, :F][near] = 0.0
    sel = np.arange(O) if nodes is None else nodes
    dx_ref, dW_ref = oracle.differentiable_lut_backward(6, x_ref, dy_ref[sel], idx[sel], W[sel], F, mean_ref[sel], rstd_ref[sel])
    dW = torch.zeros((len(sel), 64), device="cuda")
    dx = ops.differentiable_lut_backward(6, dev(x_ref), dev(dy_ref[sel]), dev(idx[sel]), dev(W[sel]), dW, F, dev(mean_ref[sel]), dev(rstd_ref[sel]),
                                         ops.reverse_table(dev(idx[sel]), I))
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F], what + " dx")
    if F <= 65536:
        assert_bwd(host(dW), dW_ref, what + " dW")
    else:
        # beyond some 10^5 frames the oracle's single fp32 accumulators (the reference's) carry more rounding than the
        # tolerance.  A float64 evaluation of the same formulas arbitrates, as in the single-layer tests: the device within
        # the tolerance of it, the oracle within a few times 1e-3.
        from test_gpu_differentiable_lut import _backward_fp64
        dW64, _ = _backward_fp64(x_ref[:, :F], dy_ref[sel][:, :F], idx[sel], W[sel], mean_ref[sel], rstd_ref[sel], GAMMA, BETA, 1)
        assert_bwd(host(dW), dW64, what + " dW against float64")
        assert rel_err(dW_ref, dW64) <= 5e-3, what + " dW of the oracle"
    if nodes is not None:
        # the whole layer on the device: the slice's table gradients are the same numbers, and dx is exactly linear in dy
        dW_all = torch.zeros((O, 64), device="cuda")
        rev = ops.reverse_table(dev(idx), I)
        dx_all = ops.differentiable_lut_backward(6, dev(x_ref), dev(dy_ref), dev(idx), dev(W), dW_all, F, dev(mean_ref), dev(rstd_ref), rev)
        assert rel_err(host(dW_all)[sel], host(dW)) <= 1e-5, what
        dW_two = torch.zeros((O, 64), device="cuda")
        dx_two = ops.differentiable_lut_backward(6, dev(x_ref), dev(dy_ref * 2.0), dev(idx), dev(W), dW_two, F, dev(mean_ref), dev(rstd_ref), rev)
        assert torch.equal(dx_two[:, :F], 2.0 * dx_all[:, :F]) and torch.equal(dW_two, 2.0 * dW_all), what
        return host(dx_all), host(dW_all)
    return dx_ref, dW_ref


def test_classifier_training_step_at_full_size():
    import torch
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    sizes = [784, 6144, 1024, 70]
    CLASSES, N_AVG, F = 10, 7, 1024
    S = synth.frame_stride_fp32(F)
    rng = np.random.default_rng(314)
    x = synth.uniform_frames(rng, sizes[0], F, S)
    label = rng.integers(0, CLASSES, F)
    t = np.zeros((CLASSES, S), F32); t[label, np.arange(F)] = 1.0
    layers = []
    for I, O in zip(sizes[:-1], sizes[1:]):
        W = np.clip(0.5 + 0.1 * rng.standard_normal((O, 64)), 0.0, 1.0).astype(F32)
        layers.append((synth.wiring(rng, I, O), W))
    idx_avg = np.arange(sizes[-1], dtype=np.int32).reshape(CLASSES, N_AVG)

    # forward, layer by layer on the oracle's activations
    a = x
    fwd = []
    for k, (idx, W) in enumerate(layers):
        y_ref, mean_ref, rstd_ref, t64 = _forward_layer(ops, a, idx, W, F, S, "layer %d" % k)
        fwd.append((a, mean_ref, rstd_ref, t64))
        a = y_ref
    # the tail: AverageLut (sum of seven 0/1 activations: exact), loss and its gradient, accuracy
    out_ref = oracle.average_lut_forward(a, idx_avg, F, False, False)
    out = ops.average_lut_forward(dev(a), dev(idx_avg), F, False, False, mean=False)
    assert np.array_equal(host(out)[:, :F], out_ref[:, :F])
    dy_ref, loss_ref, tsum_ref = oracle.loss_softmax_cross_entropy(out_ref, t, CLASSES, 1, F)
    dy, loss_buf, t_sum = ops.loss_softmax_cross_entropy(dev(out_ref), dev(t), CLASSES, 1, F)
    assert t_sum == tsum_ref
    assert abs(float(loss_buf.sum().item()) - loss_ref.sum()) <= 1e-5 * abs(loss_ref.sum())
    assert np.abs(host(dy)[:, :F] - dy_ref[:, :F]).max() * t_sum <= 2e-6
    acc, cat = ops.metrics_categorical_accuracy(dev(out_ref), dev(t), CLASSES, 1, F)
    acc_ref, cat_ref = oracle.metrics_categorical_accuracy(out_ref, t, CLASSES, 1, F)
    assert np.array_equal(host(acc), acc_ref) and np.array_equal(host(cat), cat_ref)
    g_ref = oracle.average_lut_backward(dy_ref, idx_avg, sizes[-1], F)
    g = ops.average_lut_backward(dev(dy_ref), dev(idx_avg), sizes[-1], F)
    assert np.array_equal(host(g)[:, :F], g_ref[:, :F])

    # backward, layer by layer on the oracle's gradients; then one Adam step on the oracle's table gradients
    grads = [None] * len(layers)
    for k in reversed(range(len(layers))):
        idx, W = layers[k]
        a_in, mean_ref, rstd_ref, t64 = fwd[k]
        g_ref, grads[k] = _backward_layer(ops, a_in, g_ref, idx, W, F, mean_ref, rstd_ref, t64, "layer %d" % k)
    params = [dev(W) for _, W in layers]
    adam = ops.AdamState(params, [dev(dW) for dW in grads], learning_rate=0.001)
    adam.step()
    for p, (_, W), dW in zip(params, layers, grads):
        want, _, _ = oracle.adam_steps(W.reshape(-1), [dW.reshape(-1)])
        assert np.array_equal(host(p).reshape(-1), want)


def test_conv_block_at_full_size():
    import torch
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    F, C, H, Wd, FH, FW, CO = 256, 3, 32, 32, 3, 3, 36
    OH, OW = H - FH + 1, Wd - FW + 1
    FRAMES = F * OH * OW                                        # 230 400 window frames
    S_img, S_win = synth.frame_stride_fp32(F), synth.frame_stride_fp32(FRAMES)
    rng = np.random.default_rng(2718)
    img = _pad(rng.random((C * H * Wd, F), dtype=F32), S_img)
    layers = []
    for I, O in ((C * FH * FW, 216), (216, CO)):
        layers.append((synth.wiring(rng, I, O), np.clip(0.5 + 0.1 * rng.standard_normal((O, 64)), 0.0, 1.0).astype(F32)))

    # Im2Col: a permutation, bit-exact
    cols_ref = oracle.im2col_forward(img, C, H, Wd, F, FH, FW)
    cols = ops.im2col_forward(dev(img), C, H, Wd, F, FH, FW)
    assert cols.shape == (C * FH * FW, S_win)
    assert np.array_equal(host(cols)[:, :FRAMES], cols_ref)
    # the two per-pixel layers, each on the oracle's input
    a = _pad(cols_ref, S_win)
    fwd = []
    for k, (idx, W) in enumerate(layers):
        y_ref, mean_ref, rstd_ref, t64 = _forward_layer(ops, a, idx, W, FRAMES, S_win, "conv layer %d" % k)
        fwd.append((a, mean_ref, rstd_ref, t64))
        a = y_ref
    # Col2Im and pooling on the oracle's activations: bit-exact (0/1 maps; pooling rounds each product as the host does)
    maps_ref = oracle.col2im_forward(a[:, :FRAMES], CO, OH, OW, F)
    maps = ops.col2im_forward(dev(a), CO, OH, OW, F)
    assert maps.shape == (CO * OH * OW, S_img) and np.array_equal(host(maps)[:, :F], maps_ref)
    pooled_ref = oracle.stochastic_maxpool2x2_forward(maps_ref, CO, OH, OW, F)
    pooled = ops.stochastic_maxpool2x2_forward(maps, CO, OH, OW, F)
    assert np.array_equal(host(pooled)[:, :F], pooled_ref)
    # backward: pooling, Col2Im (bit-exact), the two layers (node slices on the oracle), Im2Col (bit-exact on the same gradient)
    dpooled = rng.standard_normal((CO * (OH // 2) * (OW // 2), F)).astype(F32)
    dmaps_ref = oracle.stochastic_maxpool2x2_backward(maps_ref, dpooled, CO, OH, OW, F)
    dmaps = ops.stochastic_maxpool2x2_backward(maps, dev(_pad(dpooled, S_img)), CO, OH, OW, F)
    assert np.array_equal(host(dmaps)[:, :F], dmaps_ref)
    g_ref = oracle.col2im_backward(dmaps_ref, CO, OH, OW, F)
    g = ops.col2im_backward(dmaps, CO, OH, OW, F)
    assert g.shape == (CO, S_win) and np.array_equal(host(g)[:, :FRAMES], g_ref)
    g_ref = _pad(g_ref, S_win)
    for k in (1, 0):
        idx, W = layers[k]
        a_in, mean_ref, rstd_ref, t64 = fwd[k]
        nodes = np.linspace(0, idx.shape[0] - 1, 4).astype(np.int64)
        g_ref, _ = _backward_layer(ops, a_in, g_ref, idx, W, FRAMES, mean_ref, rstd_ref, t64, "conv layer %d" % k, nodes=nodes)
    dimg_ref = oracle.im2col_backward(g_ref[:, :FRAMES], C, H, Wd, F, FH, FW)
    dimg = ops.im2col_backward(dev(g_ref), C, H, Wd, F, FH, FW)
    assert dimg.shape == (C * H * Wd, S_img)
    # (a sum of up to nine gradients per pixel in a fixed order on both sides)
    assert np.array_equal(host(dimg)[:, :F], dimg_ref)
