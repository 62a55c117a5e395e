"""GPU parity of StochasticBatchNormalization (through the C ABI) against the CPU oracle and against the vectors that the
reference's own host class wrote (tests/golden/bn.npz).

The device sums a row lane-wise and then as a tree; the oracle and the reference sum it frame by frame.  Results therefore agree to
rounding, not bit for bit.  Tolerances, written at the assertions: statistics and y to 2e-6 + 4e-8 sqrt(F) of their scale (the
drift of a frame-order fp32 sum over F frames; the device's mean is also held to 3e-7 of the float64 mean); dx, from the oracle's own
statistics, within 1e-5 of gamma * max|dy| * rstd * max(1, max|x| * rstd), the size of the terms that cancel in it."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "bn.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _pad(a, stride, fill=0.0):
    out = np.full((a.shape[0], stride), fill, a.dtype)
    out[:, :a.shape[1]] = a
    return out


def check_forward(y, mean, rstd, rm, rv, want, x, gamma, F, momentum=0.9):
    """want: the oracle's (or the reference's) y, mean, rstd, running mean, running var.  Their frame-order fp32 sums drift by about
    sqrt(F) roundings of the running total, the device's tree sums by a few: the allowance grows with the row length, and the
    device's mean is also held to the float64 mean of the row, more tightly."""
    wy, wmean, wrstd, wrm, wrv = want
    tol = 2e-6 + 4e-8 * np.sqrt(F)
    xmax = np.abs(x[:, :F]).max(axis=1)
    assert np.all(np.abs(mean - x[:, :F].astype(np.float64).mean(axis=1)) <= 3e-7 * xmax), "mean against float64"
    assert np.all(np.abs(mean - wmean) <= tol * xmax), "mean"
    assert np.all(np.abs(rstd - wrstd) <= 2.5 * tol * wrstd), "rstd"
    assert np.all(np.abs(rm - wrm) <= tol * np.maximum(1.0, np.abs(wrm))), "running mean"
    assert np.all(np.abs(rv - wrv) <= 2.5 * tol * np.maximum(1.0, np.abs(wrv))), "running var"
    size = np.abs((x[:, :F] - wmean[:, None]) * wrstd[:, None] * gamma) + 1.0
    # a row's mean that is off by one part in 1e6 moves y by rstd * gamma * that much: the row's own scale
    slack = (xmax * wrstd * abs(gamma))[:, None]
    assert np.all(np.abs(y[:, :F] - wy[:, :F]) <= 2.5 * tol * (size + slack)), "y"


def check_backward(dx, want, dy, rstd, gamma, x, F):
    """dx = dxn rstd + dmean + x dvar / F is a sum of terms that cancel: dxn rstd is of size gamma |dy| rstd, and mean dvar / F inside
    dmean (like x dvar / F) is that times |x| rstd.  The allowance is 1e-5 of the larger of the two (with two frames, for instance,
    the output does not depend on the input at all and dx is nothing but the rounding of these terms)."""
    xmax = np.abs(x[:, :F]).max(axis=1)
    scale = (abs(gamma) * np.abs(dy[:, :F]).max(axis=1) * rstd * np.maximum(1.0, xmax * rstd))[:, None] + 1e-6
    assert np.all(np.abs(dx[:, :F].astype(np.float64) - want[:, :F]) <= 1e-5 * scale), "dx"


SHAPES = [
    # nodes, frames, stride (None: the usual padded one)
    (7, 33, None),
    (16, 128, None),
    (5, 1, None),
    (100, 4096, None),
    (11, 8192, None),           # the longest row that is kept in registers
    (3, 8193, None),            # one frame more: read once per pass
    (32, 50176, None),          # the normalisation after a convolution: 64 images of 28 x 28 positions per channel
    (9, 300, 301),              # rows that do not start on 16 bytes: one float at a time
    (4, 2048, 2049),            # the longest such row kept in registers
    (2, 2500, 2501),            # and past it
    (1000, 64, 67),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_training_backward_reforward_inference(ops, shape):
    nodes, F, stride = shape
    rng = np.random.default_rng(nodes * 131 + F)
    stride = synth.frame_stride_fp32(F) if stride is None else stride
    gamma, beta, momentum = 0.2, 0.5, 0.9
    x = _pad(rng.random((nodes, F)).astype(F32), stride)
    dy = _pad(rng.standard_normal((nodes, F)).astype(F32), stride)
    rm0 = rng.standard_normal(nodes).astype(F32); rv0 = (rng.random(nodes) + 0.5).astype(F32)

    want = oracle.stochastic_bn_forward_training(x, rm0, rv0, gamma, beta, momentum, F)
    rm = dev(rm0); rv = dev(rv0)
    y, mean, rstd = ops.stochastic_bn_forward_training(dev(x), rm, rv, F, gamma, beta, momentum)
    y, mean, rstd = host(y), host(mean), host(rstd)
    if F == 1:                          # no variance: rstd = 1e7 and y = beta exactly, on both sides
        assert np.array_equal(rstd, want[2]) and np.array_equal(y[:, :F], want[0][:, :F])
    else:
        check_forward(y, mean, rstd, host(rm), host(rv), want, x, gamma, F)

    # the other three passes from the oracle's statistics, so that each is compared on its own
    wmean, wrstd = want[1], want[2]
    yr = host(ops.stochastic_bn_reforward(dev(x), dev(wmean), dev(wrstd), F, gamma, beta))
    size = np.abs((x[:, :F] - wmean[:, None]) * wrstd[:, None] * gamma) + 1.0
    assert np.all(np.abs(yr[:, :F] - want[0][:, :F]) <= 1e-6 * size)

    yi = host(ops.stochastic_bn_forward_inference(dev(x), dev(rm0), dev(rv0), F, gamma, beta))
    wi = oracle.stochastic_bn_forward_inference(x, rm0, rv0, gamma, beta, F)
    assert np.all(np.abs(yi[:, :F] - wi[:, :F]) <= 2e-6 * (np.abs(wi[:, :F]) + 1.0))

    if F > 1:
        dx = host(ops.stochastic_bn_backward(dev(x), dev(dy), dev(wmean), dev(wrstd), F, gamma))
        check_backward(dx, oracle.stochastic_bn_backward(x, dy, wmean, wrstd, gamma, F), dy, wrstd, gamma, x, F)


def test_reference_vectors(ops):
    for k in range(int(GOLD["count"][0])):
        p = "b%d_" % k
        nodes, F = [int(v) for v in GOLD[p + "geom"]]
        momentum, gamma, beta = [float(v) for v in GOLD[p + "scalars"]]
        stride = synth.frame_stride_fp32(F)
        x = _pad(GOLD[p + "x"], stride); dy = _pad(GOLD[p + "dy"], stride)
        rm = dev(GOLD[p + "running_mean_in"]); rv = dev(GOLD[p + "running_var_in"])
        y, mean, rstd = ops.stochastic_bn_forward_training(dev(x), rm, rv, F, gamma, beta, momentum)
        y, mean, rstd = host(y), host(mean), host(rstd)
        flat = GOLD[p + "rstd"] > 1e6                      # rows without variance
        if flat.any():
            assert np.array_equal(rstd[flat], GOLD[p + "rstd"][flat]) and np.array_equal(y[flat, :F], GOLD[p + "y"][flat])
        keep = ~flat
        if keep.any():
            want = tuple(GOLD[p + key][keep] for key in ("y", "mean", "rstd", "running_mean", "running_var"))
            check_forward(y[keep], mean[keep], rstd[keep], host(rm)[keep], host(rv)[keep], want, x[keep], gamma, F)
            dx = host(ops.stochastic_bn_backward(dev(x), dev(dy), dev(GOLD[p + "mean"]), dev(GOLD[p + "rstd"]), F, gamma))
            check_backward(dx[keep], GOLD[p + "dx"][keep], dy[keep], GOLD[p + "rstd"][keep], gamma, x[keep], F)


def test_padding_is_left_alone_and_nothing_else_is_written(ops):
    import torch
    from binarybrain_amd.capi import check, lib, ptr, stream_ptr
    nodes, F, stride = 6, 70, 128
    rng = np.random.default_rng(3)
    x = dev(_pad(rng.random((nodes, F)).astype(F32), stride, fill=9.0))
    y = torch.full((nodes + 1, stride), -7.0, dtype=torch.float32, device="cuda")
    stats = torch.zeros((4, nodes + 1), dtype=torch.float32, device="cuda"); stats[:, nodes] = 5.0
    check(lib().bbhip_fp32_StochasticBatchNormalization_ForwardTraining(ptr(x), ptr(y), ptr(stats[0]), ptr(stats[1]), ptr(stats[2]),
                                                                        ptr(stats[3]), 0.2, 0.5, 0.9, nodes, F, stride, stream_ptr()))
    y = host(y); stats = host(stats)
    assert np.all(y[:nodes, F:] == -7.0) and np.all(y[nodes] == -7.0) and np.all(stats[:, nodes] == 5.0)
    want = oracle.stochastic_bn_forward_training(host(x)[:, :F].copy(), np.zeros(nodes, F32), np.zeros(nodes, F32), 0.2, 0.5, 0.9, F)
    assert np.abs(y[:nodes, :F] - want[0]).max() < 1e-5            # the 9.0 in the padding took no part in the statistics


def test_rejected_arguments(ops):
    import torch
    from binarybrain_amd import capi
    x = torch.zeros((4, 64), dtype=torch.float32, device="cuda")
    s = torch.zeros(4, dtype=torch.float32, device="cuda")
    with pytest.raises(capi.BbhipError):
        ops.stochastic_bn_forward_training(x, s, s.clone(), 65)                 # more frames than the stride
    with pytest.raises(capi.BbhipError):
        ops.stochastic_bn_forward_training(x, s, s.clone(), 0)
    with pytest.raises(capi.BbhipError):
        capi.check(capi.lib().bbhip_fp32_StochasticBatchNormalization_Backward(capi.ptr(x), None, capi.ptr(x), capi.ptr(s), capi.ptr(s),
                                                                               0.2, 1.0 / 64, 4, 64, 64, 64, capi.stream_ptr()))


def test_full_size_rows_sampled_and_invariants(ops):
    """8192 nodes x 4096 frames, the size of a hidden layer of the headline configuration: rows are independent, so the oracle
    checks a sample of them; every row is covered by what normalisation fixes (mean beta, deviation gamma, gradient sums zero)."""
    import torch
    nodes, F = 8192, 4096
    gamma, beta, momentum = 0.2, 0.5, 0.9
    g = torch.Generator(device="cuda"); g.manual_seed(7)
    x = torch.rand((nodes, F), generator=g, dtype=torch.float32, device="cuda")
    x *= torch.rand((nodes, 1), generator=g, dtype=torch.float32, device="cuda") + 0.05      # rows of different spread
    dy = torch.randn((nodes, F), generator=g, dtype=torch.float32, device="cuda")
    rm = torch.zeros(nodes, dtype=torch.float32, device="cuda"); rv = torch.ones(nodes, dtype=torch.float32, device="cuda")
    y, mean, rstd = ops.stochastic_bn_forward_training(x, rm, rv, F, gamma, beta, momentum)
    dx = ops.stochastic_bn_backward(x, dy, mean, rstd, F, gamma)
    y64 = y.double(); dx64 = dx.double()
    assert float((y64.mean(dim=1) - beta).abs().max()) < 2e-6
    assert float((y64.std(dim=1, unbiased=False) - gamma).abs().max()) < 2e-6
    scale = (dx64.abs().sum(dim=1)).clamp_min(1e-30)
    assert float((dx64.sum(dim=1).abs() / scale).max()) < 1e-5
    xc = x.double() - x.double().mean(dim=1, keepdim=True)
    assert float(((dx64 * xc).sum(dim=1).abs() / (dx64 * xc).abs().sum(dim=1).clamp_min(1e-30)).max()) < 1e-5
    rows = np.concatenate([[0, 1, nodes - 1], np.random.default_rng(1).choice(nodes, 61, replace=False)])
    xs = host(x)[rows]; dys = host(dy)[rows]
    want = oracle.stochastic_bn_forward_training(xs, np.zeros(len(rows), F32), np.ones(len(rows), F32), gamma, beta, momentum, F)
    check_forward(host(y)[rows], host(mean)[rows], host(rstd)[rows], host(rm)[rows], host(rv)[rows], want, xs, gamma, F)
    wdx = oracle.stochastic_bn_backward(xs, dys, host(mean)[rows], host(rstd)[rows], gamma, F)
    check_backward(host(dx)[rows], wdx, dys, host(rstd)[rows], gamma, xs, F)


# the grid of the reference's own fused-against-discrete test (tests/gtest/SparseLutNTest.cpp:301-403: six inputs, N = 6 and 4,
# one or two loops over fresh inputs), and one larger layer
FUSED_SHAPES = [(6, 1, 1), (6, 1, 39), (6, 1, 64), (6, 1, 1024), (6, 1024, 1), (6, 2, 32), (96, 160, 512)]


@pytest.mark.parametrize("n", [6, 4])
@pytest.mark.parametrize("binary_mode", [False, True])
@pytest.mark.parametrize("lut_binarize", [False, True])
def test_lut_then_normalisation_then_activation_is_the_differentiable_lut(ops, n, binary_mode, lut_binarize):
    """DifferentiableLutN is StochasticLutN, this normalisation and a hard-tanh activation in one layer; the reference keeps the
    three-layer form as DifferentiableLutDiscreteN (include/bb/DifferentiableLutDiscreteN.h:44-47, 271-326) and tests the fused layer
    against it (tests/gtest/SparseLutNTest.cpp:19-299; its tolerances: statistics 1e-3, rstd 0.5 %, y 1e-3, dx 0.1 absolute,
    dW 0.5 %).  Here the LUT and the normalisation are the library's entry points and the activation is written out: clamp to [0, 1]
    (binary mode: 1 where the value exceeds 0.5), gradient passed where 0 < value < 1.  The fused layer's formula differs in two
    places, which bound the agreement: it floors the variance at 1e-5 and leaves the 1e-7 out of rstd
    (include/bb/DifferentiableLutN.h:804-806).  Bars: statistics 1e-6, rstd 1e-5 relative, y 1e-5 (binary: equal outside a band of
    1e-6 around 0.5), dx and dW 1e-4 of their largest value."""
    import torch
    gamma, beta, momentum = 0.3, 0.5, 0.9
    compared = 0
    for (I, O, F) in FUSED_SHAPES:
        if I < n:
            continue
        rng = np.random.default_rng(I * 7 + O * 3 + F + n)
        stride = synth.frame_stride_fp32(F)
        idx = synth.wiring(rng, I, O, n)
        W = synth.lut_tables(rng, O, n)
        rev = ops.reverse_table(dev(idx), I)
        idxd, Wd = dev(idx), dev(W)
        rm_a = torch.zeros(O, dtype=torch.float32, device="cuda"); rv_a = torch.ones(O, dtype=torch.float32, device="cuda")
        rm_b = rm_a.clone(); rv_b = rv_a.clone()
        for loop in range(2):
            xd = dev(synth.uniform_frames(rng, I, F, stride))
            dyd = dev(_pad(rng.random((O, F)).astype(F32), stride))
            ya, mean_a, rstd_a = ops.differentiable_lut_forward_training(n, xd, idxd, Wd, F, rm_a, rv_a, gamma, beta, momentum,
                                                                         lut_binarize=lut_binarize, binary_mode=binary_mode)
            dW_a = torch.zeros_like(Wd)
            dx_a = ops.differentiable_lut_backward(n, xd, dyd, idxd, Wd, dW_a, F, mean_a, rstd_a, rev, gamma, beta,
                                                   lut_binarize=lut_binarize, binary_mode=binary_mode)

            v = ops.stochastic_lut_forward(n, xd, idxd, Wd, F, input_binary=binary_mode, lut_binarize=lut_binarize)
            t, mean_b, rstd_b = ops.stochastic_bn_forward_training(v, rm_b, rv_b, F, gamma, beta, momentum)
            yb = (t > 0.5).float() if binary_mode else t.clamp(0.0, 1.0)
            gate = ((t > 0.0) & (t < 1.0)).float()
            dv = ops.stochastic_bn_backward(v, dyd * gate, mean_b, rstd_b, F, gamma)
            dW_b = torch.zeros_like(Wd)
            dx_b = ops.stochastic_lut_backward(n, xd, dv, idxd, Wd, dW_b, F, rev, input_binary=binary_mode, lut_binarize=lut_binarize)

            case = (n, binary_mode, lut_binarize, I, O, F, loop)
            assert float((mean_a - mean_b).abs().max()) < 1e-6, case
            assert float((rm_a - rm_b).abs().max()) < 1e-6, case
            tt = host(t)[:, :F]
            # A node without variance in its batch (always so with one frame): the fused layer floors the variance, the normalisation
            # alone does not, so rstd and the running variance differ there by design; x - mean is 0 to rounding either way, both
            # write beta (to 1e-4: the floored rstd of 316 times a rounding of the mean) and pass no gradient.
            flat = host(rstd_b) > 1e6
            keep = torch.from_numpy(~flat).cuda()
            if flat.any():
                assert np.all(tt[flat] == beta) and np.all(host(dv)[:, :F][flat] == 0.0), case
            if (~flat).any():
                assert float(((rstd_a - rstd_b) / rstd_a)[keep].abs().max()) < 1e-5, case
                assert float((rv_a - rv_b)[keep].abs().max()) < 1e-6, case
            if binary_mode:
                band = np.abs(tt - 0.5) < 1e-6                         # includes every flat node: beta is 0.5
                assert np.all((host(ya)[:, :F] == host(yb)[:, :F]) | band), case
            else:
                tol = torch.from_numpy(np.where(flat, 1e-4, 1e-5).astype(F32)).cuda()[:, None]
                assert bool(((ya[:, :F] - yb[:, :F]).abs() <= tol).all()), case
            rv_b.copy_(rv_a)                                           # flat nodes: carry on from the same running variance
            # A frame whose normalised value sits within rounding of 0 or 1 may be gated on one side only, which moves the whole node's
            # gradient: such a batch is left out of the gradient comparison (binary inputs give a node only 2^n distinct values, so a
            # value on the edge repeats over many frames).
            if np.minimum(np.abs(tt), np.abs(tt - 1.0)).min() <= 1e-6:
                continue
            compared += 1
            # (flat nodes: the fused layer's floored rstd of 316 turns the rounding of its mean into gradients of about 1e-7 per node
            # where the normalisation alone passes exactly 0; an input of a thousand such nodes collects 1e-5)
            floor = 1e-4 if flat.any() else 1e-5
            for a, b, what in ((dx_a[:, :F], dx_b[:, :F], "dx"), (dW_a, dW_b, "dW")):
                assert float((a - b).abs().max()) <= 1e-4 * float(a.abs().max()) + floor, (what,) + case
    assert compared >= 10, compared                                    # of 14 batches
