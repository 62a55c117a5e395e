"""GPU parity of Im2Col / Col2Im / StochasticMaxPooling2x2 (through the C ABI) against the CPU oracle: permutations and
individually rounded products, so the bar is bit-exact everywhere."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "conv.npz"))
BORDER = {v: k for k, v in oracle.BORDER_MODES.items()}


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


IM2COL_SHAPES = [
    # c, h, w, frames, fh, fw, ys, xs, padding, border
    (2, 3, 4, 2, 2, 3, 1, 1, "valid", "reflect_101"),
    (3, 32, 32, 70, 3, 3, 1, 1, "valid", "reflect_101"),        # the benchmark's conv block geometry
    (3, 9, 11, 65, 3, 3, 1, 1, "same", "reflect_101"),
    (2, 8, 9, 3, 3, 3, 2, 2, "same", "replicate"),
    (1, 70, 5, 4, 3, 3, 2, 1, "valid", "constant"),
    (2, 6, 130, 3, 3, 5, 1, 1, "same", "wrap"),                  # more than one 64-column tile
    (2, 6, 7, 35, 3, 3, 1, 1, "same", "reflect"),
    (3, 9, 8, 3, 3, 3, 1, 2, "same", "constant"),
    (1, 1, 1, 1, 1, 1, 1, 1, "valid", "constant"),
    (32, 8, 8, 4096, 2, 1, 1, 1, "valid", "constant"),         # enough blocks for the backward kernel's 64-frame tiles
]


@pytest.mark.parametrize("shape", IM2COL_SHAPES)
def test_im2col(ops, shape):
    c, h, w, F, fh, fw, ys, xs, pad, border = shape
    rng = np.random.default_rng(abs(hash(shape)) & 0xffff)
    x = rng.random((c * h * w, F)).astype(F32)
    y_ref = oracle.im2col_forward(x, c, h, w, F, fh, fw, ys, xs, pad, border, 0.25)
    of = y_ref.shape[1]
    xs_ = _pad(x, synth.frame_stride_fp32(F))
    y = host(ops.im2col_forward(dev(xs_), c, h, w, F, fh, fw, ys, xs, pad, border, 0.25))
    assert np.array_equal(y[:, :of], y_ref)
    dy = rng.standard_normal((c * fh * fw, of)).astype(F32)
    dx_ref = oracle.im2col_backward(dy, c, h, w, F, fh, fw, ys, xs, pad)
    dx = host(ops.im2col_backward(dev(_pad(dy, synth.frame_stride_fp32(of))), c, h, w, F, fh, fw, ys, xs, pad))
    assert np.array_equal(dx[:, :F], dx_ref)
    xb = synth.bernoulli_bits(rng, c * h * w, F, synth.frame_stride_bit(F))
    yb_ref = oracle.im2col_forward(xb, c, h, w, F, fh, fw, ys, xs, pad, border, bit=True)
    yb = host(ops.im2col_forward(dev(xb), c, h, w, F, fh, fw, ys, xs, pad, border))
    assert np.array_equal(synth.unpack_bits(yb, of), synth.unpack_bits(yb_ref, of))


def test_im2col_reference_vectors(ops):
    for k in range(int(GOLD["im2col_count"][0])):
        c, h, w, F, fh, fw, ys, xs, same, border = [int(v) for v in GOLD["i%d_geom" % k]]
        pad = "same" if same else "valid"; q = "i%d_" % k
        y = host(ops.im2col_forward(dev(GOLD[q + "x"]), c, h, w, F, fh, fw, ys, xs, pad, BORDER[border]))
        of = GOLD[q + "y"].shape[1]
        assert np.array_equal(y[:, :of], GOLD[q + "y"])
        dx = host(ops.im2col_backward(dev(GOLD[q + "dy"]), c, h, w, F, fh, fw, ys, xs, pad))
        assert np.array_equal(dx[:, :F], GOLD[q + "dx"])
        yb = host(ops.im2col_forward(dev(GOLD[q + "xbits"]), c, h, w, F, fh, fw, ys, xs, pad, BORDER[border]))
        assert np.array_equal(synth.unpack_bits(yb, of), synth.unpack_bits(GOLD[q + "ybits"], of))


@pytest.mark.parametrize("shape", [(3, 4, 5, 6), (2, 1, 7, 33), (36, 30, 30, 70), (5, 9, 15, 129), (1, 1, 1, 1)])
def test_col2im(ops, shape):
    c, h, w, F = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.random((c, F * h * w)).astype(F32)
    y = host(ops.col2im_forward(dev(_pad(x, synth.frame_stride_fp32(F * h * w))), c, h, w, F))
    assert np.array_equal(y[:, :F], oracle.col2im_forward(x, c, h, w, F))
    dy = rng.standard_normal((c * h * w, F)).astype(F32)
    dx = host(ops.col2im_backward(dev(_pad(dy, synth.frame_stride_fp32(F))), c, h, w, F))
    assert np.array_equal(dx[:, :F * h * w], oracle.col2im_backward(dy, c, h, w, F))
    xb = synth.bernoulli_bits(rng, c, F * h * w, synth.frame_stride_bit(F * h * w))
    yb = host(ops.col2im_forward(dev(xb), c, h, w, F))
    assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(oracle.col2im_forward(xb, c, h, w, F, bit=True), F))


@pytest.mark.parametrize("shape", [(2, 4, 6, 5), (3, 5, 7, 9), (1, 1, 1, 3), (36, 30, 30, 300), (2, 3, 2, 1000)])
def test_stochastic_maxpool(ops, shape):
    c, h, w, F = shape
    rng = np.random.default_rng(sum(shape) + 1)
    stride = synth.frame_stride_fp32(F)
    x = _pad(rng.random((c * h * w, F)).astype(F32), stride)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    dy = _pad(rng.standard_normal((c * oh * ow, F)).astype(F32), stride)
    y = host(ops.stochastic_maxpool2x2_forward(dev(x), c, h, w, F))
    assert np.array_equal(y[:, :F], oracle.stochastic_maxpool2x2_forward(x, c, h, w, F)[:, :F])
    dx = host(ops.stochastic_maxpool2x2_backward(dev(x), dev(dy), c, h, w, F))
    assert np.array_equal(dx[:, :F], oracle.stochastic_maxpool2x2_backward(x, dy, c, h, w, F)[:, :F])


def test_conv_block_round_trip(ops):
    """Im2Col with a 1 x 1 filter followed by Col2Im gives the image back (the permutations invert each other)."""
    rng = np.random.default_rng(4)
    c, h, w, F = 3, 10, 12, 100
    img = _pad(rng.random((c * h * w, F)).astype(F32), synth.frame_stride_fp32(F))
    cols = ops.im2col_forward(dev(img), c, h, w, F, 1, 1)
    back = host(ops.col2im_forward(cols, c, h, w, F))
    assert np.array_equal(back[:, :F], img[:, :F])


def test_rejects_bad_arguments(ops):
    from binarybrain_amd import capi
    lib = capi.lib()
    assert lib.bbhip_fp32_Col2Im_Forward(None, None, 2, 2, 2, 16, 4, 4, None) != 0
    assert lib.bbhip_fp32_StochasticMaxPooling2x2_Forward(None, None, 4, 4, 2, 2, 1, 8, 8, None) != 0
    import torch
    t = torch.zeros(64, device="cuda")
    p = capi.ptr(t)
    assert lib.bbhip_fp32_StochasticMaxPooling2x2_Forward(p, p, 4, 4, 3, 2, 1, 1, 1, None) != 0       # wrong output size
    assert lib.bbhip_fp32_Im2Col_Forward(p, p, 1, 1, 0, 0, 1, 1, 4, 4, 1, 2, 2, 4, 3, 3, 7, 0.0, None) != 0   # unknown border mode
    assert lib.bbhip_fp32_Im2Col_Forward(p, p, 1, 1, 0, 0, 1, 1, 4, 4, 1, 2, 2, 3, 3, 3, 0, 0.0, None) != 0   # output stride too short
