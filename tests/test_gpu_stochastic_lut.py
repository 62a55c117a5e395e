"""GPU parity of the StochasticLut entry points (through the C ABI) against the CPU oracle.

Shapes follow the reference's own parity test (tests/gtest/StochasticLutNTest.cpp:235-246) plus the CPU-runnable
benchmark configuration (784 -> 1024 nodes, 64 frames) and ragged frame counts.
"""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import assert_bwd, assert_fwd, dev, host, rel_err

pytestmark = pytest.mark.gpu

REF_SHAPES = [(6, 1, 1), (14, 16, 8), (14, 1024, 8), (14, 1024, 3), (13, 17, 1529), (784, 1024, 64), (40, 33, 300)]


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    yield o
    o.set_dx_mode(0)


def _case(rng, n, I, O, F, lo=-0.1, hi=1.1):
    stride = synth.frame_stride_fp32(F)
    idx = synth.wiring(rng, I, O, n)
    W = oracle.vector_clamp(synth.lut_tables(rng, O, n, -0.2, 1.2))
    x = synth.uniform_frames(rng, I, F, stride, lo, hi)
    dy = synth.normal_frames(rng, O, F, stride)
    return stride, idx, W, x, dy


@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("lut_binarize", [0, 1])
@pytest.mark.parametrize("input_binary", [0, 1])
def test_lut6_forward_backward(ops, shape, lut_binarize, input_binary):
    I, O, F = shape
    rng = np.random.default_rng(hash((I, O, F, lut_binarize, input_binary)) & 0xffff)
    stride, idx, W, x, dy = _case(rng, 6, I, O, F)
    dW0 = rng.standard_normal((O, 64)).astype(np.float32)
    y_ref = oracle.stochastic_lut_forward(6, x, idx, W, F, input_binary, lut_binarize, 0.25, F % 8 == 0)
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, x, dy, idx, W, F, dW0, input_binary, lut_binarize, 0.25, F % 8 == 0)

    y = ops.stochastic_lut_forward(6, dev(x), dev(idx), dev(W), F, input_binary, lut_binarize)
    assert_fwd(host(y)[:, :F], y_ref[:, :F], "y")
    rev = ops.reverse_table(dev(idx), I)
    assert np.array_equal(host(rev), oracle.reverse_table(6, idx, I))
    for mode in (0, 1, 2):
        ops.set_dx_mode(mode)
        dW = dev(dW0.copy())
        dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, input_binary, lut_binarize)
        assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "dx mode %d" % mode)
        assert_bwd(host(dW), dW_ref, "dW mode %d" % mode)
    ops.set_dx_mode(0)


@pytest.mark.parametrize("F", [700, 200])     # several units per node (the table launch clamps); one (the wavefronts clamp their node's table)
@pytest.mark.parametrize("n,input_binary,lut_binarize", [(6, 0, 0), (6, 1, 0), (6, 0, 1), (4, 0, 0), (2, 1, 1)])
def test_forward_that_clamps_the_table_in_place(ops, n, input_binary, lut_binarize, F):
    """bbhip_fp32_StochasticLut_ForwardClampW = bbhip_fp32_Vector_clamp on W + bbhip_fp32_StochasticLut_Forward, bit for bit
    (what StochasticLutN::Forward does before every pass, include/bb/StochasticLutN.h:451): W afterwards equals the oracle's
    clamp, y equals the forward pass on the clamped table; a table already inside the range is left untouched."""
    rng = np.random.default_rng(77 + n)
    I, O = 40, 37
    stride = synth.frame_stride_fp32(F)
    idx = synth.wiring(rng, I, O, n)
    W0 = synth.lut_tables(rng, O, n, -0.3, 1.3)
    x = synth.uniform_frames(rng, I, F, stride, -0.1, 1.1)
    for lo, hi in ((0.0, 1.0), (0.25, 0.5)):
        W = dev(W0.copy())
        y = ops.stochastic_lut_forward(n, dev(x), dev(idx), W, F, input_binary, lut_binarize, clamp_w=(lo, hi))
        Wc = oracle.vector_clamp(W0, lo, hi)
        assert np.array_equal(host(W), Wc)
        y2 = ops.stochastic_lut_forward(n, dev(x), dev(idx), dev(Wc), F, input_binary, lut_binarize)
        assert np.array_equal(host(y)[:, :F], host(y2)[:, :F])
        assert_fwd(host(y)[:, :F], oracle.stochastic_lut_forward(n, x, idx, Wc, F, input_binary, lut_binarize, 0.25, False)[:, :F], "y")
        # a second call finds nothing to clamp and writes nothing back
        y3 = ops.stochastic_lut_forward(n, dev(x), dev(idx), W, F, input_binary, lut_binarize, clamp_w=(lo, hi))
        assert np.array_equal(host(W), Wc) and np.array_equal(host(y3)[:, :F], host(y)[:, :F])
    with pytest.raises(RuntimeError):
        ops.stochastic_lut_forward(n, dev(x), dev(idx), dev(W0.copy()), F, input_binary, lut_binarize, clamp_w=(1.0, 0.0))


@pytest.mark.parametrize("n", [2, 3, 4, 5])
def test_other_widths(ops, n):
    rng = np.random.default_rng(100 + n)
    for (I, O, F) in [(12, 9, 70), (30, 64, 256)]:
        for lut_binarize in (0, 1):
            stride, idx, W, x, dy = _case(rng, n, I, O, F)
            y_ref = oracle.stochastic_lut_forward(n, x, idx, W, F, 0, lut_binarize, 0.25, False)
            dx_ref, dW_ref = oracle.stochastic_lut_backward(n, x, dy, idx, W, F, None, 0, lut_binarize, 0.25, False)
            y = ops.stochastic_lut_forward(n, dev(x), dev(idx), dev(W), F, False, lut_binarize)
            assert_fwd(host(y)[:, :F], y_ref[:, :F])
            rev = ops.reverse_table(dev(idx), I)
            for mode in (0, 1, 2):
                ops.set_dx_mode(mode)
                dW = dev(np.zeros((O, 1 << n), np.float32))
                dx = ops.stochastic_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, False, lut_binarize)
                assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)
    ops.set_dx_mode(0)


@pytest.mark.parametrize("n", [6, 4, 2])
def test_bit_input(ops, n):
    rng = np.random.default_rng(200 + n)
    for (I, O, F) in [(24, 16, 70), (64, 40, 2048 + 33)]:
        for lut_binarize in (0, 1):
            idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
            xs = synth.frame_stride_bit(F); ys = synth.frame_stride_fp32(F)
            xb = synth.bernoulli_bits(rng, I, F, xs); dy = synth.normal_frames(rng, O, F, ys)
            y_ref = oracle.bit_stochastic_lut_forward(n, xb, idx, W, F, ys, lut_binarize)
            dx_ref, dW_ref = oracle.bit_stochastic_lut_backward(n, xb, dy, idx, W, F, None, lut_binarize)
            yb_ref = oracle.bit_bit_stochastic_lut_forward(n, xb, idx, W, F, lut_binarize)
            y = ops.bit_stochastic_lut_forward(n, dev(xb), dev(idx), dev(W), F, ys, lut_binarize)
            assert_fwd(host(y)[:, :F], y_ref[:, :F])
            yb = ops.bit_bit_stochastic_lut_forward(n, dev(xb), dev(idx), dev(W), F, lut_binarize)
            # inputs take two values, so the LUT output takes at most 2^n values per node: a threshold flip needs an
            # exact tie at 0.5, which random tables do not produce -> bit-exact
            assert np.array_equal(synth.unpack_bits(host(yb), F), synth.unpack_bits(yb_ref, F))
            rev = ops.reverse_table(dev(idx), I)
            for mode in (0, 1, 2):
                ops.set_dx_mode(mode)
                dW = dev(np.zeros((O, 1 << n), np.float32))
                dx = ops.bit_stochastic_lut_backward(n, dev(xb), dev(dy), dev(idx), dev(W), dW, F, rev, lut_binarize)
                assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)
    ops.set_dx_mode(0)


@pytest.mark.parametrize("extra_words", [1, 3, 8])
def test_bit_input_row_pitches(ops, extra_words):
    """packed rows whose pitch is not a multiple of 8 words take the per-step loads, others the 32-byte loads: same results"""
    rng = np.random.default_rng(300 + extra_words)
    I, O, F = 40, 24, 1000
    idx = synth.wiring(rng, I, O, 6); W = synth.lut_tables(rng, O, 6)
    xs = (F + 31) // 32 + extra_words; ys = synth.frame_stride_fp32(F)
    xb = synth.bernoulli_bits(rng, I, F, xs); dy = synth.normal_frames(rng, O, F, ys)
    y_ref = oracle.bit_stochastic_lut_forward(6, xb, idx, W, F, ys, 0)
    y = ops.bit_stochastic_lut_forward(6, dev(xb), dev(idx), dev(W), F, ys, 0)
    assert_fwd(host(y)[:, :F], y_ref[:, :F])
    yb = ops.bit_bit_stochastic_lut_forward(6, dev(xb), dev(idx), dev(W), F, 0)
    assert np.array_equal(synth.unpack_bits(host(yb), F), synth.unpack_bits(oracle.bit_bit_stochastic_lut_forward(6, xb, idx, W, F, 0), F))
    dx_ref, dW_ref = oracle.bit_stochastic_lut_backward(6, xb, dy, idx, W, F, None, 0)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.bit_stochastic_lut_backward(6, dev(xb), dev(dy), dev(idx), dev(W), dW, F, ops.reverse_table(dev(idx), I), 0)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)


@pytest.mark.parametrize("stride", [1001, 1002, 1004])
def test_binarized_input_row_pitches(ops, stride):
    """binary mode on fp32 frames: the backward pass packs the binarized input, four frames per lane where the row pitch
    allows 16-byte loads and frame by frame elsewhere: same results"""
    rng = np.random.default_rng(400 + stride)
    I, O, F = 40, 24, 1000
    idx = synth.wiring(rng, I, O, 6); W = synth.lut_tables(rng, O, 6)
    x = synth.uniform_frames(rng, I, F, stride); dy = synth.normal_frames(rng, O, F, stride)
    y_ref = oracle.stochastic_lut_forward(6, x, idx, W, F, 1, 0, 0.25, False)
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, x, dy, idx, W, F, None, 1, 0, 0.25, False)
    y = ops.stochastic_lut_forward(6, dev(x), dev(idx), dev(W), F, True, False)
    assert_fwd(host(y)[:, :F], y_ref[:, :F])
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, ops.reverse_table(dev(idx), I), True, False)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)


def test_golden_vectors_on_gpu(ops):
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "stochastic_lut.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        n, I, O, F, simd, binary_mode, lut_binarize = [int(v) for v in g[p + "meta"]]
        if simd < 0:
            continue
        stride = synth.frame_stride_fp32(F)
        x = np.zeros((I, stride), np.float32); x[:, :F] = g[p + "x"]
        dy = np.zeros((O, stride), np.float32); dy[:, :F] = g[p + "dy"]
        W = dev(g[p + "W"])
        ops.vector_clamp_(W)
        assert np.array_equal(host(W), g[p + "Wc"])
        y = ops.stochastic_lut_forward(n, dev(x), dev(g[p + "idx"]), W, F, binary_mode, lut_binarize)
        assert_fwd(host(y)[:, :F], g[p + "y"])
        dW = dev(g[p + "dW0"])
        rev = ops.reverse_table(dev(g[p + "idx"]), I)
        dx = ops.stochastic_lut_backward(n, dev(x), dev(dy), dev(g[p + "idx"]), W, dW, F, rev, binary_mode, lut_binarize)
        assert_bwd(host(dx)[:, :F], g[p + "dx"]); assert_bwd(host(dW), g[p + "dW"])


def test_tmp_chunking_and_determinism(ops):
    rng = np.random.default_rng(5)
    I, O, F = 50, 37, 1000
    stride, idx, W, x, dy = _case(rng, 6, I, O, F)
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, x, dy, idx, W, F, None, 0, 0, 0.25, True)
    rev = ops.reverse_table(dev(idx), I)
    # mode 2 with a dx_tmp smaller than the frame range: the frames are walked in several passes
    ops.set_dx_mode(2)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, max_tmp_bytes=4 * O * 6 * 96)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F]); assert_bwd(host(dW), dW_ref)
    # the deterministic modes are reproducible bit for bit
    for mode in (0, 2):
        ops.set_dx_mode(mode)
        outs = []
        for _ in range(2):
            dW = dev(np.zeros((O, 64), np.float32))
            dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev)
            outs.append((host(dx)[:, :F].copy(), host(dW).copy()))
        assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    ops.set_dx_mode(0)
    # an input node nobody reads gets dx = 0
    idx2 = idx.copy(); idx2[idx2 == 7] = 8
    for o in range(O):                       # keep the 6 inputs of a node distinct
        while len(set(idx2[o])) < 6:
            idx2[o] = synth.wiring(rng, I, 1)[0]; idx2[o][idx2[o] == 7] = 9
    rev2 = ops.reverse_table(dev(idx2), I)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx2), dev(W), dW, F, rev2)
    if not (idx2 == 7).any():
        assert np.array_equal(host(dx)[7, :F], np.zeros(F, np.float32))


def test_rejected_arguments(ops):
    import torch
    from binarybrain_amd.capi import BbhipError
    x = torch.zeros((8, 64), device="cuda"); idx = torch.zeros((4, 6), dtype=torch.int32, device="cuda")
    W = torch.zeros((4, 64), device="cuda")
    with pytest.raises(BbhipError):
        ops.stochastic_lut_forward(7, x, idx, W, 64)            # width outside 2..6
    with pytest.raises(BbhipError):
        ops.stochastic_lut_forward(6, x, idx, W, 65)            # stride shorter than the frames
    with pytest.raises(BbhipError):
        ops.stochastic_lut_forward(6, x, idx, W, 0)             # empty frame range
    ops.set_dx_mode(0)
    with pytest.raises(BbhipError):                              # deterministic dx without a reverse table
        ops.stochastic_lut_backward(6, x, x[:4].contiguous(), idx, W, torch.zeros_like(W), 64, rev=None)


def test_full_size_properties(ops):
    """4096 -> 4096 nodes, 8192 frames: the oracle checks a slice of nodes; size-independent rules check the rest."""
    import torch
    rng = np.random.default_rng(42)
    I = O = 4096; F = 8192
    idx = synth.wiring(rng, I, O); W = synth.lut_tables(rng, O)
    x = synth.uniform_frames(rng, I, F, F); dy = synth.normal_frames(rng, O, F, F)
    xd, dyd, idxd, Wd = dev(x), dev(dy), dev(idx), dev(W)
    y = ops.stochastic_lut_forward(6, xd, idxd, Wd, F)
    sel = np.arange(0, O, 64)
    y_ref = oracle.stochastic_lut_forward(6, x, idx[sel], W[sel], F)
    assert_fwd(host(y)[sel], y_ref)
    ops.set_dx_mode(1)
    dW = torch.zeros((O, 64), device="cuda")
    dx = ops.stochastic_lut_backward(6, xd, dyd, idxd, Wd, dW, F)
    # sum_i prod_i = 1  =>  sum_i dW[o, i] = sum_f dy[o, f]
    s = dy.astype(np.float64).sum(1)
    assert np.abs(host(dW).astype(np.float64).sum(1) - s).max() <= 1e-4 * np.abs(s).max()
    # dW of the selected nodes against the oracle (dW of a node depends on that node only)
    _, dW_ref = oracle.stochastic_lut_backward(6, x, dy[sel], idx[sel], W[sel], F)
    assert_bwd(host(dW)[sel], dW_ref)
    # dx: deterministic and atomic accumulation agree, dx is linear in dy, and a slice of frames matches the oracle
    ops.set_dx_mode(0)
    rev = ops.reverse_table(idxd, I)
    dWb = torch.zeros((O, 64), device="cuda")
    dxb = ops.stochastic_lut_backward(6, xd, dyd, idxd, Wd, dWb, F, rev)
    assert rel_err(host(dx), host(dxb)) <= 1e-5 and rel_err(host(dW), host(dWb)) <= 1e-5
    dWc = torch.zeros((O, 64), device="cuda")
    dxc = ops.stochastic_lut_backward(6, xd, (dyd * 2.0).contiguous(), idxd, Wd, dWc, F, rev)
    assert rel_err(host(dxc), 2.0 * host(dxb)) <= 1e-6
    fs = 256
    dx_ref, _ = oracle.stochastic_lut_backward(6, np.ascontiguousarray(x[:, :fs]), np.ascontiguousarray(dy[:, :fs]), idx, W, fs)
    assert_bwd(host(dxb)[:, :fs], dx_ref)
    # every node: y over a 512-frame slice in the middle of the batch, and dW of the full-size call when dy is zero outside that
    # slice (then the table gradient is that of the slice alone, and so is dx inside it)
    f0, fn = 4096 + 64, 512
    xs_, dys_ = np.ascontiguousarray(x[:, f0:f0 + fn]), np.ascontiguousarray(dy[:, f0:f0 + fn])
    assert_fwd(host(y)[:, f0:f0 + fn], oracle.stochastic_lut_forward(6, xs_, idx, W, fn))
    dy_cut = np.zeros_like(dy); dy_cut[:, f0:f0 + fn] = dys_
    dWs = torch.zeros((O, 64), device="cuda")
    dxs = ops.stochastic_lut_backward(6, xd, dev(dy_cut), idxd, Wd, dWs, F, rev)
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, xs_, dys_, idx, W, fn)
    assert_bwd(host(dWs), dW_ref)
    assert_bwd(host(dxs)[:, f0:f0 + fn], dx_ref)
    assert not host(dxs)[:, :f0].any() and not host(dxs)[:, f0 + fn:].any()


def test_full_size_properties_packed_bits(ops):
    """4096 -> 4096 nodes, 8192 frames of packed bits (the lookup kernels for two-valued inputs at their full shape): a slice of
    nodes and a slice of frames against the oracle, the fp32 entry point on the unpacked 0/1 frames in binary mode, linearity"""
    import torch
    rng = np.random.default_rng(43)
    I = O = 4096; F = 8192
    idx = synth.wiring(rng, I, O); W = synth.lut_tables(rng, O)
    xs = synth.frame_stride_bit(F); ys = synth.frame_stride_fp32(F)
    xb = synth.bernoulli_bits(rng, I, F, xs); dy = synth.normal_frames(rng, O, F, ys)
    xd, dyd, idxd, Wd = dev(xb), dev(dy), dev(idx), dev(W)
    ops.set_dx_mode(0)
    y = ops.bit_stochastic_lut_forward(6, xd, idxd, Wd, F, ys, 0)
    sel = np.arange(0, O, 64)
    assert_fwd(host(y)[sel][:, :F], oracle.bit_stochastic_lut_forward(6, xb, idx[sel], W[sel], F, ys, 0)[:, :F])
    rev = ops.reverse_table(idxd, I)
    dW = torch.zeros((O, 64), device="cuda")
    dx = ops.bit_stochastic_lut_backward(6, xd, dyd, idxd, Wd, dW, F, rev, 0)
    s = dy[:, :F].astype(np.float64).sum(1)
    assert np.abs(host(dW).astype(np.float64).sum(1) - s).max() <= 1e-4 * np.abs(s).max()
    _, dW_ref = oracle.bit_stochastic_lut_backward(6, xb, dy[sel], idx[sel], W[sel], F, None, 0)
    assert_bwd(host(dW)[sel], dW_ref)
    # the same frames as fp32 0 / 1 values through the fp32 entry points in binary mode
    xf = np.zeros((I, ys), np.float32); xf[:, :F] = synth.unpack_bits(xb, F)
    yf = ops.stochastic_lut_forward(6, dev(xf), idxd, Wd, F, True, False)
    assert rel_err(host(yf)[:, :F], host(y)[:, :F]) <= 1e-6
    dWf = torch.zeros((O, 64), device="cuda")
    dxf = ops.stochastic_lut_backward(6, dev(xf), dyd, idxd, Wd, dWf, F, rev, True, False)
    assert rel_err(host(dxf)[:, :F], host(dx)[:, :F]) <= 1e-6 and rel_err(host(dWf), host(dW)) <= 1e-6
    # linear in dy, and a slice of frames against the oracle
    dWc = torch.zeros((O, 64), device="cuda")
    dxc = ops.bit_stochastic_lut_backward(6, xd, (dyd * 2.0).contiguous(), idxd, Wd, dWc, F, rev, 0)
    assert rel_err(host(dxc)[:, :F], 2.0 * host(dx)[:, :F]) <= 1e-6          # (the padding of a row is not written)
    fs = 256
    dx_ref, _ = oracle.bit_stochastic_lut_backward(6, np.ascontiguousarray(xb[:, :fs // 32]), np.ascontiguousarray(dy[:, :fs]), idx, W, fs, None, 0)
    assert_bwd(host(dx)[:, :fs], dx_ref)


def _adversarial_tables(n):
    """Tables whose monomial coefficients are as large as a [0,1] table allows: parity, AND, OR, single spikes."""
    nn = 1 << n
    i = np.arange(nn)
    pop = np.array([bin(v).count("1") for v in i])
    t = [
        (pop & 1).astype(np.float32),                 # parity: plain-basis coefficients (-2)^(|S|-1)
        1.0 - (pop & 1).astype(np.float32),
        (i == nn - 1).astype(np.float32),             # AND
        (i != 0).astype(np.float32),                  # OR
        np.ones(nn, np.float32),
        np.zeros(nn, np.float32),
        ((i >> (n - 1)) & 1).astype(np.float32),      # projection on the last input
        (i == 5 % nn).astype(np.float32),             # one spike
    ]
    return np.stack(t)


@pytest.mark.parametrize("n", [6, 5, 4, 3, 2])
def test_adversarial_tables(ops, n):
    """Worst cases for a monomial-basis evaluation: extreme tables with inputs at and near the corners of the cube.
    The oracle here is the defining formula in fp64 (sum of 2^n products), not an fp32 association."""
    rng = np.random.default_rng(700 + n)
    T = _adversarial_tables(n)
    O = T.shape[0] * 4
    I, F = 16, 192
    W = np.tile(T, (4, 1)).astype(np.float32)
    idx = synth.wiring(rng, I, O, n)
    stride = synth.frame_stride_fp32(F)
    x = np.zeros((I, stride), np.float32)
    x[:, :64] = rng.integers(0, 2, (I, 64)).astype(np.float32)                     # corners
    x[:, 64:128] = np.clip(rng.integers(0, 2, (I, 64)) + rng.normal(0, 1e-3, (I, 64)), 0, 1)   # next to corners
    x[:, 128:F] = rng.random((I, F - 128))
    dy = synth.normal_frames(rng, O, F, stride)

    xs = x[idx][:, :, :F].astype(np.float64)                                       # [O][n][F]
    y64 = np.zeros((O, F)); dW64 = np.zeros((O, 1 << n)); dx64 = np.zeros((I, F))
    for i in range(1 << n):
        fac = [xs[:, j] if (i >> j) & 1 else 1.0 - xs[:, j] for j in range(n)]
        prod = np.prod(fac, axis=0)
        y64 += W[:, i:i + 1] * prod
        dW64[:, i] = (dy[:, :F] * prod).sum(axis=1)
        for j in range(n):
            others = np.prod([fac[k] for k in range(n) if k != j], axis=0) if n > 1 else 1.0
            g = W[:, i:i + 1] * others * dy[:, :F] * (1.0 if (i >> j) & 1 else -1.0)
            np.add.at(dx64, idx[:, j], g)

    y = ops.stochastic_lut_forward(n, dev(x), dev(idx), dev(W), F, False, False)
    assert_fwd(host(y)[:, :F], np.clip(y64, 0, 1), "y")
    rev = ops.reverse_table(dev(idx), I)
    for mode in (0, 1, 2):
        ops.set_dx_mode(mode)
        dW = dev(np.zeros((O, 1 << n), np.float32))
        dx = ops.stochastic_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, False, False)
        assert_bwd(host(dx)[:, :F], dx64, "dx mode %d" % mode)
        assert_bwd(host(dW), dW64, "dW mode %d" % mode)
    ops.set_dx_mode(0)
    # the exact corner frames reproduce the table entries themselves
    corner = host(y)[:, :64]
    sel = (xs[:, :, :64] > 0.5).astype(np.int64)
    code = sum(sel[:, j] << j for j in range(n))
    assert np.array_equal(corner, np.take_along_axis(W, code, axis=1))


def test_skewed_fan_out_takes_another_dx_path():
    """One input that feeds every node makes the reverse table input_nodes x (1 + output_nodes) wide, far more slots than
    connections: the deterministic dx kernel's term table would be sized by that, so the library takes the dx_tmp scheme
    (when given the buffer) or the atomic one for such a call.  Results stay within the backward tolerance."""
    import torch
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    rng = np.random.default_rng(4242)
    I, O, F = 3000, 400, 200
    S = synth.frame_stride_fp32(F)
    idx = synth.wiring(rng, I - 1, O, 6) + 1
    idx[:, 2] = 0                                   # input 0 is wired to every node
    W = synth.lut_tables(rng, O); x = synth.uniform_frames(rng, I, F, S, -0.1, 1.1); dy = synth.normal_frames(rng, O, F, S)
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, x, dy, idx, W, F)
    rev = ops.reverse_table(dev(idx), I)
    assert rev.shape[1] == O + 1
    for with_tmp in (False, True):
        dW = torch.zeros((O, 64), device="cuda")
        kw = dict(dx_tmp=torch.empty((O * 6, S), device="cuda"), tmp_frame_size=F) if with_tmp else {}
        dx = ops.stochastic_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, **kw)
        assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "dx"); assert_bwd(host(dW), dW_ref, "dW")
