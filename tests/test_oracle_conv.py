"""The oracle's Im2Col / Col2Im / StochasticMaxPooling2x2, pinned without a GPU: vectors written by the reference's own
host classes (tests/golden/conv.npz), the compiled reference where oracle/_ref is present, the known answers of the
reference's tests (tests/gtest/ConvolutionIm2ColTest.cpp:19-232) restated here, and identities of the permutations."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "conv.npz"))
BORDER = {v: k for k, v in oracle.BORDER_MODES.items()}
F32 = np.float32


def im2col_gold(k):
    c, h, w, F, fh, fw, ys, xs, same, border = [int(v) for v in GOLD["i%d_geom" % k]]
    return dict(c=c, h=h, w=w, frames=F, fh=fh, fw=fw, ys=ys, xs=xs, padding="same" if same else "valid", border=BORDER[border])


def test_im2col_reference_vectors():
    for k in range(int(GOLD["im2col_count"][0])):
        g = im2col_gold(k); q = "i%d_" % k
        y = oracle.im2col_forward(GOLD[q + "x"], **g)
        assert np.array_equal(y, GOLD[q + "y"]), g
        gb = {n: v for n, v in g.items() if n != "border"}
        assert np.array_equal(oracle.im2col_backward(GOLD[q + "dy"], **gb), GOLD[q + "dx"]), g
        yb = oracle.im2col_forward(GOLD[q + "xbits"], bit=True, **g)
        of = y.shape[1]
        assert np.array_equal(synth.unpack_bits(yb, of), synth.unpack_bits(GOLD[q + "ybits"], of)), g


def test_im2col_known_answers_of_the_reference_test():
    # testConvolutionIm2Col: 2 frames of {2, 3, 4}, value 1000 f + 100 c + 10 y + x, filter 2 x 3, valid
    c, h, w, F, fh, fw = 2, 3, 4, 2, 2, 3
    x = np.zeros((c * h * w, F), F32)
    for f in range(F):
        for cc in range(c):
            for yy in range(h):
                for xx in range(w):
                    x[(cc * h + yy) * w + xx, f] = 1000 * f + 100 * cc + 10 * yy + xx
    y = oracle.im2col_forward(x, c, h, w, F, fh, fw)
    node = lambda cc, yy, xx: (cc * fh + yy) * fw + xx
    for frame, base in [(0, 0), (1, 1), (2, 10), (3, 11), (6, 1010), (7, 1011)]:      # ConvolutionIm2ColTest.cpp:40-116
        for cc in range(c):
            for yy in range(fh):
                for xx in range(fw):
                    assert y[node(cc, yy, xx), frame] == base + 100 * cc + 10 * yy + xx
    dy = np.zeros((c * fh * fw, 8), F32)
    for f in range(8):
        for cc in range(c):
            for yy in range(fh):
                for xx in range(fw):
                    dy[node(cc, yy, xx), f] = 1000 * f + 100 * cc + 10 * yy + xx
    dx = oracle.im2col_backward(dy, c, h, w, F, fh, fw)
    d = lambda f, cc, yy, xx: dy[node(cc, yy, xx), f]
    for f in range(F):                                                             # :133-189
        for cc in range(c):
            n = lambda yy, xx: (cc * h + yy) * w + xx
            assert dx[n(0, 0), f] == d(f * 4, cc, 0, 0)
            assert dx[n(0, 1), f] == d(f * 4, cc, 0, 1) + d(f * 4 + 1, cc, 0, 0)
            assert dx[n(0, 3), f] == d(f * 4 + 1, cc, 0, 2)
            assert dx[n(1, 1), f] == d(f * 4, cc, 1, 1) + d(f * 4 + 1, cc, 1, 0) + d(f * 4 + 2, cc, 0, 1) + d(f * 4 + 3, cc, 0, 0)
            assert dx[n(1, 3), f] == d(f * 4 + 1, cc, 1, 2) + d(f * 4 + 3, cc, 0, 2)
            assert dx[n(2, 3), f] == d(f * 4 + 3, cc, 1, 2)
    # testConvolutionIm2Col_float: 3 x 3 image 011/101/010, filter 2 x 2                 :194-232
    img = np.array([0, 1, 1, 1, 0, 1, 0, 1, 0], F32).reshape(9, 1)
    y = oracle.im2col_forward(img, 1, 3, 3, 1, 2, 2)
    assert y.T.tolist() == [[0, 1, 1, 0], [1, 1, 0, 1], [1, 0, 0, 1], [0, 1, 1, 0]]
    yb = oracle.im2col_forward(synth.pack_bits(img.astype(np.uint8), 1), 1, 3, 3, 1, 2, 2, bit=True)
    assert synth.unpack_bits(yb, 4).T.tolist() == [[0, 1, 1, 0], [1, 1, 0, 1], [1, 0, 0, 1], [0, 1, 1, 0]]


def test_im2col_backward_is_the_transpose_of_forward():
    """<Im2Col(x), dy> == <x, Im2Col^T(dy)> wherever no border replica is read (valid padding, or constant border)."""
    rng = np.random.default_rng(3)
    for (c, h, w, F, fh, fw, ys, xs, pad) in [(2, 6, 5, 3, 3, 3, 1, 1, "valid"), (1, 9, 7, 2, 3, 2, 2, 2, "valid"), (2, 6, 6, 2, 3, 3, 1, 1, "same")]:
        x = rng.standard_normal((c * h * w, F)).astype(F32)
        y = oracle.im2col_forward(x, c, h, w, F, fh, fw, ys, xs, pad, "constant", 0.0)
        dy = rng.standard_normal(y.shape).astype(F32)
        dx = oracle.im2col_backward(dy, c, h, w, F, fh, fw, ys, xs, pad)
        assert abs(float((y.astype(np.float64) * dy).sum()) - float((x.astype(np.float64) * dx).sum())) < 1e-3


def test_col2im_vectors_and_inverse():
    for k in range(int(GOLD["col2im_count"][0])):
        c, h, w, F = [int(v) for v in GOLD["c%d_geom" % k]]; q = "c%d_" % k
        y = oracle.col2im_forward(GOLD[q + "x"], c, h, w, F)
        assert np.array_equal(y, GOLD[q + "y"])
        assert np.array_equal(oracle.col2im_backward(GOLD[q + "dy"], c, h, w, F), GOLD[q + "dx"])
        assert np.array_equal(oracle.col2im_backward(y, c, h, w, F), GOLD[q + "x"])           # backward inverts forward
        yb = oracle.col2im_forward(GOLD[q + "xbits"], c, h, w, F, bit=True)
        assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(GOLD[q + "ybits"], F))
    # written independently: y[(c, xy)][f] = x[c][f*hw + xy] is a reshape + transpose
    rng = np.random.default_rng(1)
    x = rng.random((3, 5 * 12)).astype(F32)
    assert np.array_equal(oracle.col2im_forward(x, 3, 3, 4, 5), x.reshape(3, 5, 12).transpose(0, 2, 1).reshape(36, 5))
    # Im2Col followed by a 1 x 1 "convolution" and Col2Im is the identity on images
    img = rng.random((2 * 4 * 5, 3)).astype(F32)
    cols = oracle.im2col_forward(img, 2, 4, 5, 3, 1, 1)
    assert np.array_equal(oracle.col2im_forward(cols, 2, 4, 5, 3), img)


def test_pooling_vectors_and_closed_form():
    for k in range(int(GOLD["pool_count"][0])):
        c, h, w, F = [int(v) for v in GOLD["p%d_geom" % k]]; q = "p%d_" % k
        assert np.array_equal(oracle.stochastic_maxpool2x2_forward(GOLD[q + "x"], c, h, w, F), GOLD[q + "y"])
        assert np.array_equal(oracle.stochastic_maxpool2x2_backward(GOLD[q + "x"], GOLD[q + "dy"], c, h, w, F), GOLD[q + "dx"])
    rng = np.random.default_rng(2)
    c, h, w, F = 2, 4, 6, 7
    x = rng.random((c * h * w, F))
    y = oracle.stochastic_maxpool2x2_forward(x, c, h, w, F)
    x4 = x.reshape(c, h // 2, 2, w // 2, 2, F)
    assert np.allclose(y.reshape(c, h // 2, w // 2, F), 1 - np.prod(1 - x4, axis=(2, 4)), atol=2e-7)     # probabilistic OR
    bits = (x > 0.5).astype(F32)
    assert np.array_equal(oracle.stochastic_maxpool2x2_forward(bits, c, h, w, F).reshape(c, h // 2, w // 2, F),
                          bits.reshape(c, h // 2, 2, w // 2, 2, F).max(axis=(2, 4)))                      # binary inputs: max
    eps = 1e-3
    dy = rng.standard_normal(y.shape).astype(F32)
    dx = oracle.stochastic_maxpool2x2_backward(x, dy, c, h, w, F)
    xp = x.copy(); xp[5, 2] += eps; xm = x.copy(); xm[5, 2] -= eps
    num = ((oracle.stochastic_maxpool2x2_forward(xp, c, h, w, F).astype(np.float64) - oracle.stochastic_maxpool2x2_forward(xm, c, h, w, F)) * dy).sum() / (2 * eps)
    assert abs(num - dx[5, 2]) < 2e-3


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (reference tree absent)")
def test_against_compiled_reference():
    rng = np.random.default_rng(9)
    for (c, h, w, F, fh, fw, ys, xs, pad, border) in [(2, 7, 9, 4, 3, 3, 1, 1, "same", "reflect_101"), (1, 10, 6, 3, 5, 3, 2, 1, "valid", "constant"),
                                                      (2, 5, 5, 33, 3, 3, 1, 1, "same", "wrap"), (2, 8, 8, 2, 3, 3, 2, 2, "same", "reflect")]:
        x = rng.random((c * h * w, F)).astype(F32)
        y = oracle.im2col_forward(x, c, h, w, F, fh, fw, ys, xs, pad, border)
        dy = rng.standard_normal(y.shape).astype(F32)
        yr, dxr = oracle.ref_im2col(x, c, h, w, F, fh, fw, ys, xs, pad, border, dy=dy)
        assert np.array_equal(y, yr) and np.array_equal(oracle.im2col_backward(dy, c, h, w, F, fh, fw, ys, xs, pad), dxr)
    x = rng.random((4, 10 * 6)).astype(F32)
    assert np.array_equal(oracle.col2im_forward(x, 4, 2, 3, 10), oracle.ref_col2im(x, 4, 2, 3, 10)[0])
    x = rng.random((3 * 7 * 5, 6)).astype(F32); dy = rng.standard_normal((3 * 4 * 3, 6)).astype(F32)
    yr, dxr = oracle.ref_stochastic_maxpool2x2(x, 3, 7, 5, 6, dy=dy)
    assert np.array_equal(oracle.stochastic_maxpool2x2_forward(x, 3, 7, 5, 6), yr)
    assert np.array_equal(oracle.stochastic_maxpool2x2_backward(x, dy, 3, 7, 5, 6), dxr)


def test_col2im_known_answers_of_the_reference_test():
    # testConvolutionCol2ImTest (tests/gtest/ConvolutionCol2ImTest.cpp:9-90): 2 channels, 2 frames of 3 x 4 pixels,
    # value 1000 f + 100 c + 10 y + x at frame (f*3 + y)*4 + x of channel c goes to pixel (c, y, x) of frame f
    c, h, w, F = 2, 3, 4, 2
    x = np.zeros((c, F * h * w), F32)
    for f in range(F):
        for yy in range(h):
            for xx in range(w):
                for cc in range(c):
                    x[cc, (f * h + yy) * w + xx] = 1000 * f + 100 * cc + 10 * yy + xx
    y = oracle.col2im_forward(x, c, h, w, F)
    for f in range(F):
        for cc in range(c):
            for yy in range(h):
                for xx in range(w):
                    assert y[(cc * h + yy) * w + xx, f] == 1000 * f + 100 * cc + 10 * yy + xx
    assert np.array_equal(oracle.col2im_backward(y, c, h, w, F), x)
