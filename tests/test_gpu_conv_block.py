"""The convolutional LUT block end to end on the GPU (Im2Col 3 x 3 -> DifferentiableLut6 27 -> 216 -> 36 per pixel with
batch-norm in binary mode -> Col2Im -> StochasticMaxPooling2x2, forward and backward down to the image gradient), at a
reduced image size and batch, against the same chain of CPU oracle calls.  Every piece has its own parity test; this one
checks that they compose: shapes, row pitches and frame orders handed from one entry point to the next.

Binarized activations may differ from the oracle's where a pre-activation sits within rounding of the threshold, so each
GPU layer is also fed the oracle's own input and compared on that (exact up to such frames), and the chain as a whole is
compared through the fraction of differing activations and the relative error of the gradients."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
C, H, W, FH, FW, CO = 3, 12, 10, 3, 3, 36
OH, OW = H - FH + 1, W - FW + 1
F = 24                                   # images
FRAMES = F * OH * OW                     # window frames of the per-pixel layers


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


def test_conv_block_chain():
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    rng = np.random.default_rng(31)
    S_img, S_win = synth.frame_stride_fp32(F), synth.frame_stride_fp32(FRAMES)
    img = _pad(rng.random((C * H * W, F)).astype(F32), S_img)
    dpooled = rng.standard_normal((CO * (OH // 2) * (OW // 2), F)).astype(F32)
    layers = []
    for I, O in ((C * FH * FW, 216), (216, CO)):
        idx = synth.wiring(rng, I, O)
        Wt = (0.5 + 0.1 * rng.standard_normal((O, 64))).astype(F32)
        layers.append((I, O, idx, Wt))

    # ---- oracle chain (dense rows) ----
    a = oracle.im2col_forward(img, C, H, W, F, FH, FW)
    ref = {"cols": a}
    acts = []
    for k, (I, O, idx, Wt) in enumerate(layers):
        y, mean, rstd, _, _ = oracle.differentiable_lut_forward_training(6, a, idx, Wt, FRAMES, np.zeros(O, F32), np.ones(O, F32))
        acts.append((a, mean, rstd)); a = y
        ref["y%d" % k] = y
    ref["maps"] = oracle.col2im_forward(a, CO, OH, OW, F)
    ref["pooled"] = oracle.stochastic_maxpool2x2_forward(ref["maps"], CO, OH, OW, F)
    dy = oracle.col2im_backward(oracle.stochastic_maxpool2x2_backward(ref["maps"], dpooled, CO, OH, OW, F), CO, OH, OW, F)
    for k in (1, 0):
        I, O, idx, Wt = layers[k]
        a_in, mean, rstd = acts[k]
        dy, dW = oracle.differentiable_lut_backward(6, a_in, dy, idx, Wt, FRAMES, mean, rstd)
        ref["dW%d" % k] = dW
    ref["dimg"] = oracle.im2col_backward(dy, C, H, W, F, FH, FW)

    # ---- the same chain through the C ABI ----
    import torch
    cols = ops.im2col_forward(dev(img), C, H, W, F, FH, FW)
    assert cols.shape == (C * FH * FW, S_win)
    assert np.array_equal(host(cols)[:, :FRAMES], ref["cols"])
    a = cols; gacts = []; dWs = []
    for k, (I, O, idx, Wt) in enumerate(layers):
        y, mean, rstd = ops.differentiable_lut_forward_training(6, a, dev(idx), dev(Wt), FRAMES, torch.zeros(O, device="cuda"), torch.ones(O, device="cuda"))
        gacts.append((a, mean, rstd)); a = y
        assert np.mean(host(y)[:, :FRAMES] != ref["y%d" % k]) < 2e-3, k
        # the layer on the oracle's own input: only threshold ties may differ
        y_own, _, _ = ops.differentiable_lut_forward_training(6, dev(_pad(acts[k][0], S_win)), dev(idx), dev(Wt), FRAMES,
                                                              torch.zeros(O, device="cuda"), torch.ones(O, device="cuda"))
        assert np.mean(host(y_own)[:, :FRAMES] != ref["y%d" % k]) < 2e-4, k
    maps = ops.col2im_forward(a, CO, OH, OW, F)
    assert maps.shape == (CO * OH * OW, S_img)
    pooled = ops.stochastic_maxpool2x2_forward(maps, CO, OH, OW, F)
    assert np.mean(np.abs(host(pooled)[:, :F] - ref["pooled"]) > 1e-6) < 5e-3
    dmaps = ops.stochastic_maxpool2x2_backward(maps, dev(_pad(dpooled, S_img)), CO, OH, OW, F)
    dy = ops.col2im_backward(dmaps, CO, OH, OW, F)
    assert dy.shape == (CO, S_win)
    for k in (1, 0):
        I, O, idx, Wt = layers[k]
        a_in, mean, rstd = gacts[k]
        dW = torch.zeros((O, 64), device="cuda")
        dy = ops.differentiable_lut_backward(6, a_in, dy, dev(idx), dev(Wt), dW, FRAMES, mean, rstd, ops.reverse_table(dev(idx), I))
        err = np.abs(host(dW) - ref["dW%d" % k]).max() / np.abs(ref["dW%d" % k]).max()
        assert err < 3e-2, (k, err)
    dimg = host(ops.im2col_backward(dy, C, H, W, F, FH, FW))
    assert dimg.shape == (C * H * W, S_img)
    err = np.abs(dimg[:, :F] - ref["dimg"]).max() / np.abs(ref["dimg"]).max()
    assert err < 3e-2, err
