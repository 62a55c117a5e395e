"""GPU parity of the DifferentiableLut entry points (LUT fused with per-node batch-norm and binarize / hard-tanh).

Frame counts follow the reference's fused-vs-discrete test (tests/gtest/SparseLutNTest.cpp: 1, 39, 64, 1024, 32, 131).
Binarized outputs may legitimately flip where the pre-threshold value is within rounding of 0.5; such frames are
identified with an fp64 evaluation and excluded (their number is bounded).
"""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import assert_bwd, dev, host, rel_err

pytestmark = pytest.mark.gpu

FRAMES = [1, 39, 64, 1024, 32, 131, 2048 + 17]     # (the last: several units per node, ragged last pass)


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    yield o
    o.set_dx_mode(0)


def _pre_activation(n, xc, idx, W, mean, rstd, gamma, beta):
    """fp64 value of ((LUT - mean) * rstd) * gamma + beta for centred-and-mapped inputs xc [I, F]"""
    xs = xc.astype(np.float64)[idx]
    raw = np.zeros((idx.shape[0], xc.shape[1]))
    for i in range(1 << n):
        raw += W[:, i:i + 1].astype(np.float64) * np.prod([xs[:, j] if (i >> j) & 1 else 1 - xs[:, j] for j in range(n)], axis=0)
    return (raw - mean[:, None]) * rstd[:, None] * gamma + beta


def _check_binary(y_gpu, y_ref, pre, what):
    diff = (y_gpu != y_ref)
    near = np.abs(pre - 0.5) < 2e-6
    assert not (diff & ~near).any(), "%s: %d mismatches away from the threshold" % (what, int((diff & ~near).sum()))
    assert diff.sum() <= max(2, 1e-4 * diff.size)


@pytest.mark.parametrize("n", [6, 4, 2])
@pytest.mark.parametrize("F", FRAMES)
def test_fp32_training_inference_backward(ops, n, F):
    rng = np.random.default_rng(1000 * n + F)
    I, O = 24, 20
    gamma, beta, mom = 0.3, 0.5, 0.9
    stride = synth.frame_stride_fp32(F)
    for (binary_mode, lut_binarize) in [(1, 0), (0, 0), (1, 1)]:
        idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
        x = synth.uniform_frames(rng, I, F, stride, -0.1, 1.1); dy = synth.normal_frames(rng, O, F, stride)
        rm = rng.random(O).astype(np.float32); rv = (rng.random(O) + 0.5).astype(np.float32)
        y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.differentiable_lut_forward_training(
            n, x, idx, W, F, rm, rv, gamma, beta, mom, 0.25, lut_binarize, binary_mode)
        rmd, rvd = dev(rm), dev(rv)
        y, mean, rstd = ops.differentiable_lut_forward_training(n, dev(x), dev(idx), dev(W), F, rmd, rvd, gamma, beta, mom,
                                                                0.25, lut_binarize, binary_mode)
        assert rel_err(host(mean), mean_ref) <= 1e-5 and rel_err(host(rstd), rstd_ref) <= 1e-4      # reference tolerance: 1e-3 / 0.5 %
        assert rel_err(host(rmd), rm_ref) <= 1e-5 and rel_err(host(rvd), rv_ref) <= 1e-5
        Wb = (W > 0.5).astype(np.float32) if lut_binarize else W
        xc = np.where(x > 0.5, 0.75, 0.25).astype(np.float32) if binary_mode else np.clip(x, 0, 1)
        if binary_mode:
            pre = _pre_activation(n, xc[:, :F], idx, Wb, mean_ref.astype(np.float64), rstd_ref.astype(np.float64), gamma, beta)
            _check_binary(host(y)[:, :F], y_ref[:, :F], pre, "train y")
        else:
            # the output scales with rstd (up to 316 when the variance floor 1e-5 is hit): tolerance relative to gamma*rstd
            tol = 1e-5 * np.maximum(1.0, gamma * rstd_ref)[:, None]
            assert (np.abs(host(y)[:, :F] - y_ref[:, :F]) <= tol).all()

        # inference uses the running statistics
        yi_ref = oracle.differentiable_lut_forward_inference(n, x, idx, W, F, rm_ref, rv_ref, gamma, beta, 0.25, lut_binarize, binary_mode)
        yi = ops.differentiable_lut_forward_inference(n, dev(x), dev(idx), dev(W), F, dev(rm_ref), dev(rv_ref), gamma, beta, 0.25,
                                                      lut_binarize, binary_mode)
        if binary_mode:
            pre = _pre_activation(n, xc[:, :F], idx, Wb, rm_ref.astype(np.float64), 1 / np.sqrt(rv_ref.astype(np.float64)), gamma, beta)
            _check_binary(host(yi)[:, :F], yi_ref[:, :F], pre, "inference y")
        else:
            assert np.abs(host(yi)[:, :F] - yi_ref[:, :F]).max() <= 1e-5

        # backward from the oracle's statistics
        dx_ref, dW_ref = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, mean_ref, rstd_ref, None, gamma, beta, 0.25,
                                                            lut_binarize, binary_mode)
        rev = ops.reverse_table(dev(idx), I)
        for mode in (0, 1, 2):
            ops.set_dx_mode(mode)
            dW = dev(np.zeros((O, 1 << n), np.float32))
            dx = ops.differentiable_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, dev(mean_ref), dev(rstd_ref), rev,
                                                 gamma, beta, 0.25, lut_binarize, binary_mode)
            if np.abs(dx_ref).max() > 0:
                assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "dx mode %d" % mode)
                assert_bwd(host(dW), dW_ref, "dW mode %d" % mode)
            else:       # a single frame: the batch statistics remove the whole gradient
                assert np.abs(host(dx)[:, :F]).max() <= 1e-5 and np.abs(host(dW)).max() <= 1e-5
        ops.set_dx_mode(0)


@pytest.mark.parametrize("n", [6, 4])
def test_larger_layer(ops, n):
    """one 784 -> 1024 layer at batch 1024 (first layer shape class of the MLP configuration)"""
    rng = np.random.default_rng(77 + n)
    I, O, F = 784, 256, 1024
    stride = F
    idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
    x = synth.uniform_frames(rng, I, F, stride); dy = synth.normal_frames(rng, O, F, stride)
    rm = np.zeros(O, np.float32); rv = np.ones(O, np.float32)
    for binary_mode in (1, 0):
        y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, binary_mode=binary_mode)
        rmd, rvd = dev(rm), dev(rv)
        y, mean, rstd = ops.differentiable_lut_forward_training(n, dev(x), dev(idx), dev(W), F, rmd, rvd, binary_mode=binary_mode)
        assert rel_err(host(mean), mean_ref) <= 1e-5 and rel_err(host(rstd), rstd_ref) <= 1e-4
        if binary_mode:
            assert (host(y) != y_ref).mean() <= 1e-4
        else:
            assert np.abs(host(y) - y_ref).max() <= 1e-4
        dx_ref, dW_ref = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, mean_ref, rstd_ref, binary_mode=binary_mode)
        rev = ops.reverse_table(dev(idx), I)
        dW = dev(np.zeros((O, 1 << n), np.float32))
        dx = ops.differentiable_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, mean, rstd, rev, binary_mode=binary_mode)
        assert_bwd(host(dx), dx_ref); assert_bwd(host(dW), dW_ref)


def _backward_fp64(x, dy, idx, W, mean, rstd, gamma, beta, binary_mode):
    """fp64 evaluation of DifferentiableLut6's backward with batch-norm (include/bb/DifferentiableLutN.h:1157-1266) for
    the table gradient: the gradient behind the hard-tanh window, the batch-norm backward from the stored statistics,
    then dW[i] = sum_f d * prod_j(x_j or 1 - x_j).  Also returns the batch-norm output t [O, F], which decides the window."""
    F = x.shape[1]
    dW = np.zeros((idx.shape[0], 64)); t_all = np.zeros((idx.shape[0], F))
    for o in range(idx.shape[0]):
        xs = x[idx[o]].astype(np.float64)
        xs = np.where(xs > 0.5, 0.75, 0.25) if binary_mode else np.clip(xs, 0.0, 1.0)
        p = np.ones((64, F))
        for i in range(64):
            for j in range(6):
                p[i] *= xs[j] if (i >> j) & 1 else 1.0 - xs[j]
        v = W[o].astype(np.float64) @ p
        m, r = float(mean[o]), float(rstd[o])
        t = ((v - m) * r) * gamma + beta
        g = np.where((t > 0.0) & (t < 1.0), dy[o].astype(np.float64), 0.0) * gamma
        dstd = -(g * (v - m) * r * r).sum(); dmeanx = -(g * r).sum()
        dvar = dstd * r; dmean = (dmeanx - m * dvar) / F
        dW[o] = p @ (g * r + dmean + v * dvar / F)
        t_all[o] = t
    return dW, t_all


def _layer_at_full_shape(ops, I, O, F, binary_mode, slice_nodes):
    """A layer at a shape of the reference's configurations.  Nodes are independent in everything but dx, and batch-norm
    couples all frames of a node, so the oracle (whose backward is a single-threaded loop, as the reference's) checks a
    layer made of a slice of the nodes over all frames: y, statistics, dW and the slice's dx.  The full layer is
    checked against that slice, and its dx through rules that hold at any size: exactly linear in dy under a factor of
    two, the same in all three accumulation modes."""
    import torch
    rng = np.random.default_rng(I * O + binary_mode)
    stride = synth.frame_stride_fp32(F)
    idx = synth.wiring(rng, I, O); W = synth.lut_tables(rng, O)
    x = synth.uniform_frames(rng, I, F, stride); dy = synth.normal_frames(rng, O, F, stride)
    sel = np.linspace(0, O - 1, slice_nodes).astype(np.int64)
    seld = torch.from_numpy(sel).cuda()
    xd, dyd, idxd, Wd = dev(x), dev(dy), dev(idx), dev(W)
    rm = np.zeros(O, np.float32); rv = np.ones(O, np.float32)
    y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.differentiable_lut_forward_training(6, x, idx[sel], W[sel], F, rm[sel], rv[sel],
                                                                                           binary_mode=binary_mode)
    rmd, rvd = dev(rm), dev(rv)
    y, mean, rstd = ops.differentiable_lut_forward_training(6, xd, idxd, Wd, F, rmd, rvd, binary_mode=binary_mode)
    assert rel_err(host(mean)[sel], mean_ref) <= 1e-5 and rel_err(host(rstd)[sel], rstd_ref) <= 1e-4
    assert rel_err(host(rmd)[sel], rm_ref) <= 1e-5 and rel_err(host(rvd)[sel], rv_ref) <= 1e-5
    if binary_mode:
        assert (host(y)[sel][:, :F] != y_ref[:, :F]).mean() <= 1e-4
    else:
        assert (np.abs(host(y)[sel][:, :F] - y_ref[:, :F]) <= 1e-5 * np.maximum(1.0, 0.3 * rstd_ref)[:, None]).all()
    # The gradient passes a frame only where the batch-norm output t lies inside (0, 1).  Among a million (node, frame)
    # pairs a few have t within rounding of an edge, and which side fp32 puts them on is not part of the contract: dy is
    # zeroed for those pairs of the checked nodes, so that both sides pass nothing there.
    _, t64 = _backward_fp64(x[:, :F], dy[sel][:, :F], idx[sel], W[sel], mean_ref, rstd_ref, 0.3, 0.5, binary_mode)
    near = (np.abs(t64) < 1e-5) | (np.abs(t64 - 1.0) < 1e-5)
    assert near.sum() <= 1e-3 * near.size
    for k, o in enumerate(sel):
        dy[o, :F][near[k]] = 0.0
    dyd = dev(dy)
    # the slice as a layer of its own: dx and dW against the oracle over all frames
    dx_ref, dW_ref = oracle.differentiable_lut_backward(6, x, dy[sel], idx[sel], W[sel], F, mean_ref, rstd_ref, binary_mode=binary_mode)
    ops.set_dx_mode(0)
    rev_sel = ops.reverse_table(dev(idx[sel]), I)
    dW_sel = torch.zeros((len(sel), 64), device="cuda")
    dx_sel = ops.differentiable_lut_backward(6, xd, dev(dy[sel]), dev(idx[sel]), dev(W[sel]), dW_sel, F, dev(mean_ref), dev(rstd_ref),
                                             rev_sel, binary_mode=binary_mode)
    assert_bwd(host(dx_sel)[:, :F], dx_ref[:, :F], "dx of the slice")
    if F <= 65536:
        assert_bwd(host(dW_sel), dW_ref, "dW of the slice")
    else:
        # The oracle adds the F terms of a table gradient, and of the two batch-norm sums behind every one of them, in
        # one fp32 accumulator each, as the reference does; beyond some 10^5 frames its own rounding reaches the
        # tolerance.  An fp64 evaluation of the same formulas is the arbiter: the device within the tolerance, the
        # oracle within ten times that.
        dW64, _ = _backward_fp64(x[:, :F], dy[sel][:, :F], idx[sel], W[sel], mean_ref, rstd_ref, 0.3, 0.5, binary_mode)
        assert_bwd(host(dW_sel), dW64, "dW of the slice against fp64")
        assert rel_err(dW_ref, dW64) <= 1e-3
    # the full layer, from the device's own statistics; the slice again from the same statistics
    rev = ops.reverse_table(idxd, I)
    dW = torch.zeros((O, 64), device="cuda")
    dx = ops.differentiable_lut_backward(6, xd, dyd, idxd, Wd, dW, F, mean, rstd, rev, binary_mode=binary_mode)
    dW_own = torch.zeros((len(sel), 64), device="cuda")
    ops.differentiable_lut_backward(6, xd, dev(dy[sel]), dev(idx[sel]), dev(W[sel]), dW_own, F, mean[seld].contiguous(),
                                    rstd[seld].contiguous(), rev_sel, binary_mode=binary_mode)
    assert rel_err(host(dW)[sel], host(dW_own)) <= 1e-5            # the two launches divide the frames differently
    dW2 = torch.zeros((O, 64), device="cuda")
    dx2 = ops.differentiable_lut_backward(6, xd, (dyd * 2.0).contiguous(), idxd, Wd, dW2, F, mean, rstd, rev, binary_mode=binary_mode)
    assert torch.equal(dx2[:, :F], 2.0 * dx[:, :F]) and torch.equal(dW2, 2.0 * dW)
    for mode in (1, 2):
        ops.set_dx_mode(mode)
        dWm = torch.zeros((O, 64), device="cuda")
        dxm = ops.differentiable_lut_backward(6, xd, dyd, idxd, Wd, dWm, F, mean, rstd, rev, binary_mode=binary_mode)
        assert rel_err(host(dxm)[:, :F], host(dx)[:, :F]) <= 1e-5 and rel_err(host(dWm), host(dW)) <= 1e-5
    ops.set_dx_mode(0)


@pytest.mark.parametrize("shape", [(784, 6144, 256), (6144, 1024, 256), (1024, 70, 70)])
def test_classifier_layers_at_full_shape(ops, shape):
    """the three layers of the MNIST-like classifier at its batch of 1024 frames (binary mode, the class default)"""
    I, O, slice_nodes = shape
    _layer_at_full_shape(ops, I, O, 1024, 1, slice_nodes)


@pytest.mark.parametrize("shape", [(27, 216, 1), (216, 36, 1), (216, 36, 0)])
def test_conv_block_layers_at_full_shape(ops, shape):
    """the two per-pixel layers of the convolutional configuration at their 230 400 frames (256 images of 30 x 30 pixels)"""
    I, O, binary_mode = shape
    _layer_at_full_shape(ops, I, O, 230400, binary_mode, 4)


@pytest.mark.parametrize("n", [6, 4])
def test_bit_variants(ops, n):
    rng = np.random.default_rng(300 + n)
    for (I, O, F) in [(24, 16, 70), (64, 40, 1024), (30, 9, 2048 + 17)]:
        for lut_binarize in (0, 1):
            idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
            xs = synth.frame_stride_bit(F); ys = synth.frame_stride_fp32(F)
            xb = synth.bernoulli_bits(rng, I, F, xs); dy = synth.normal_frames(rng, O, F, ys)
            rm = rng.random(O).astype(np.float32); rv = (rng.random(O) + 0.5).astype(np.float32)
            y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.bit_differentiable_lut_forward_training(n, xb, idx, W, F, rm, rv, lut_binarize=lut_binarize)
            rmd, rvd = dev(rm), dev(rv)
            y, mean, rstd = ops.bit_differentiable_lut_forward_training(n, dev(xb), dev(idx), dev(W), F, rmd, rvd, lut_binarize=lut_binarize)
            assert rel_err(host(mean), mean_ref) <= 1e-5 and rel_err(host(rstd), rstd_ref) <= 1e-4
            assert rel_err(host(rmd), rm_ref) <= 1e-5 and rel_err(host(rvd), rv_ref) <= 1e-5
            yg = synth.unpack_bits(host(y), F); yr = synth.unpack_bits(y_ref, F)
            Wb = (W > 0.5).astype(np.float32) if lut_binarize else W
            xc = np.where(synth.unpack_bits(xb, F) > 0, 0.75, 0.25)
            pre = _pre_activation(n, xc, idx, Wb, mean_ref.astype(np.float64), rstd_ref.astype(np.float64), 0.3, 0.5)
            _check_binary(yg, yr, pre, "bit train")
            # padding bits of the last word are written as zero
            assert np.array_equal(host(y) & ~synth.pack_bits(np.ones((O, F), np.uint8), xs), np.zeros_like(y_ref))
            yi_ref = oracle.bit_differentiable_lut_forward_inference(n, xb, idx, W, F, rm_ref, rv_ref, lut_binarize=lut_binarize)
            yi = ops.bit_differentiable_lut_forward_inference(n, dev(xb), dev(idx), dev(W), F, dev(rm_ref), dev(rv_ref), lut_binarize=lut_binarize)
            pre = _pre_activation(n, xc, idx, Wb, rm_ref.astype(np.float64), 1 / np.sqrt(rv_ref.astype(np.float64)), 0.3, 0.5)
            _check_binary(synth.unpack_bits(host(yi), F), synth.unpack_bits(yi_ref, F), pre, "bit inference")
            dx_ref, dW_ref = oracle.bit_differentiable_lut_backward(n, xb, dy, idx, W, F, mean_ref, rstd_ref, lut_binarize=lut_binarize)
            rev = ops.reverse_table(dev(idx), I)
            for mode in (0, 1, 2):
                ops.set_dx_mode(mode)
                dW = dev(np.zeros((O, 1 << n), np.float32))
                dx = ops.bit_differentiable_lut_backward(n, dev(xb), dev(dy), dev(idx), dev(W), dW, F, dev(mean_ref), dev(rstd_ref), rev,
                                                         lut_binarize=lut_binarize)
                assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)
            ops.set_dx_mode(0)


@pytest.mark.parametrize("n", [6, 3])
def test_training_forward_that_clamps_the_table_in_place(ops, n):
    """The ...ForwardTrainingClampW entries = bbhip_fp32_Vector_clamp on W + the ForwardTraining entry, bit for bit (the model
    class clamps its table before the first forward pass after a backward pass, include/bb/DifferentiableLutN.h:605-608):
    W afterwards equals the oracle's clamp; outputs, statistics and running statistics equal those of the two-call form."""
    rng = np.random.default_rng(900 + n)
    I, O, F = 48, 41, 1100
    idx = synth.wiring(rng, I, O, n)
    W0 = synth.lut_tables(rng, O, n, -0.3, 1.3)
    Wc = oracle.vector_clamp(W0, 0.0, 1.0)
    ys = synth.frame_stride_fp32(F)
    x = synth.uniform_frames(rng, I, F, ys)
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
    rm = rng.random(O).astype(np.float32); rv = (rng.random(O) + 0.5).astype(np.float32)
    for binary_mode in (True, False):
        W = dev(W0.copy()); rm1, rv1 = dev(rm), dev(rv); rm2, rv2 = dev(rm), dev(rv)
        y1, m1, r1 = ops.differentiable_lut_forward_training(n, dev(x), dev(idx), W, F, rm1, rv1, binary_mode=binary_mode, clamp_w=(0.0, 1.0))
        y2, m2, r2 = ops.differentiable_lut_forward_training(n, dev(x), dev(idx), dev(Wc), F, rm2, rv2, binary_mode=binary_mode)
        assert np.array_equal(host(W), Wc)
        for a, b in ((y1[:, :F], y2[:, :F]), (m1, m2), (r1, r2), (rm1, rm2), (rv1, rv2)):
            assert np.array_equal(host(a), host(b))
    W = dev(W0.copy()); rm1, rv1 = dev(rm), dev(rv); rm2, rv2 = dev(rm), dev(rv)
    y1, m1, r1 = ops.bit_differentiable_lut_forward_training(n, dev(xb), dev(idx), W, F, rm1, rv1, clamp_w=(0.0, 1.0))
    y2, m2, r2 = ops.bit_differentiable_lut_forward_training(n, dev(xb), dev(idx), dev(Wc), F, rm2, rv2)
    assert np.array_equal(host(W), Wc)
    for a, b in ((y1, y2), (m1, m2), (r1, r2), (rm1, rm2), (rv1, rv2)):
        assert np.array_equal(host(a), host(b))


@pytest.mark.parametrize("n", [6, 4])
def test_no_batchnorm_forward(ops, n):
    rng = np.random.default_rng(400 + n)
    I, O, F = 20, 16, 77
    stride = synth.frame_stride_fp32(F)
    idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
    x = synth.uniform_frames(rng, I, F, stride, -0.1, 1.1)
    for binary_mode in (0, 1):
        y_ref = oracle.differentiable_lut_forward_nobn(n, x, idx, W, F, binary_mode=binary_mode)
        y = ops.differentiable_lut_forward_nobn(n, dev(x), dev(idx), dev(W), F, binary_mode=binary_mode)
        if binary_mode:
            assert (host(y)[:, :F] != y_ref[:, :F]).sum() <= 1
        else:
            assert np.abs(host(y)[:, :F] - y_ref[:, :F]).max() <= 1e-5


def test_golden_vectors_on_gpu(ops):
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "differentiable_lut.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        n, I, O, F, bit, binary_mode, lut_binarize, batch_norm = [int(v) for v in g[p + "meta"]]
        if bit or not batch_norm:
            continue
        stride = synth.frame_stride_fp32(F)
        x = np.zeros((I, stride), np.float32); x[:, :F] = g[p + "x"]
        dy = np.zeros((O, stride), np.float32); dy[:, :F] = g[p + "dy"]
        rmd, rvd = dev(g[p + "rm"]), dev(g[p + "rv"])
        y, mean, rstd = ops.differentiable_lut_forward_training(n, dev(x), dev(g[p + "idx"]), dev(g[p + "W"]), F, rmd, rvd,
                                                                lut_binarize=lut_binarize, binary_mode=binary_mode)
        assert rel_err(host(mean), g[p + "mean"]) <= 1e-5 and rel_err(host(rstd), g[p + "rstd"]) <= 1e-4
        assert rel_err(host(rmd), g[p + "rm_out"]) <= 1e-5 and rel_err(host(rvd), g[p + "rv_out"]) <= 1e-5
        if binary_mode:
            assert (host(y)[:, :F] != g[p + "y"]).sum() <= 2
        else:
            tol = 1e-5 * np.maximum(1.0, 0.3 * g[p + "rstd"])[:, None]
            assert (np.abs(host(y)[:, :F] - g[p + "y"]) <= tol).all()
        dW = dev(np.zeros((O, 1 << n), np.float32))
        rev = ops.reverse_table(dev(g[p + "idx"]), I)
        dx = ops.differentiable_lut_backward(n, dev(x), dev(dy), dev(g[p + "idx"]), dev(g[p + "W"]), dW, F, dev(g[p + "mean"]),
                                             dev(g[p + "rstd"]), rev, lut_binarize=lut_binarize, binary_mode=binary_mode)
        assert_bwd(host(dx)[:, :F], g[p + "dx"]); assert_bwd(host(dW), g[p + "dW"])
