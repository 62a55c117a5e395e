"""The oracle's MaxPooling and UpSampling, pinned without a GPU: vectors written by the reference's own host classes
(tests/golden/pooling.npz), the compiled reference where oracle/_ref is present, the known answers of the reference's tests
(tests/gtest/MaxPoolingTest.cpp:9-146, UpSamplingTest.cpp:21-120) and numpy.  Selections and sums in a fixed order: bit-exact."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "pooling.npz"))
F32 = np.float32


def test_reference_vectors():
    for k in range(int(GOLD["pool_count"][0])):
        q = "p%d_" % k
        c, h, w, fh, fw, F = [int(v) for v in GOLD[q + "geom"]]
        y, arg = oracle.max_pooling_forward(GOLD[q + "x"], c, h, w, fh, fw, F)
        assert np.array_equal(y, GOLD[q + "y"]), k
        assert np.array_equal(oracle.max_pooling_backward(arg, GOLD[q + "dy"], c, h, w, fh, fw, F), GOLD[q + "dx"]), k
        assert np.array_equal(oracle.bit_max_pooling_forward(GOLD[q + "xbits"], c, h, w, fh, fw, F), GOLD[q + "y_bits"]), k
        assert np.array_equal(oracle.bit_max_pooling_backward(GOLD[q + "xbits"], GOLD[q + "dy"], c, h, w, fh, fw, F), GOLD[q + "dx_from_bits"]), k
    for k in range(int(GOLD["up_count"][0])):
        q = "u%d_" % k
        c, h, w, fh, fw, fill, F = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(oracle.up_sampling_forward(GOLD[q + "x"], c, h, w, fh, fw, F, bool(fill)), GOLD[q + "y"]), k
        assert np.array_equal(oracle.up_sampling_backward(GOLD[q + "dy"], c, h, w, fh, fw, F, bool(fill)), GOLD[q + "dx"]), k
        assert np.array_equal(oracle.up_sampling_forward(GOLD[q + "xbits"], c, h, w, fh, fw, F, bool(fill), bit=True), GOLD[q + "y_bits"]), k


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_against_compiled_reference():
    rng = np.random.default_rng(61)
    for (c, h, w, fh, fw, F) in [(3, 7, 9, 2, 2, 37), (1, 4, 4, 4, 4, 64), (5, 6, 6, 3, 2, 5), (2, 9, 5, 2, 3, 100)]:
        x = rng.standard_normal((c * h * w, F)).astype(F32)
        x[rng.random(x.shape) < 0.3] = 0.25
        O = c * ((h + fh - 1) // fh) * ((w + fw - 1) // fw)
        dy = rng.standard_normal((O, F)).astype(F32)
        y, arg = oracle.max_pooling_forward(x, c, h, w, fh, fw, F)
        yr, dxr, _ = oracle.ref_max_pooling(x, c, h, w, fh, fw, F, dy=dy)
        assert np.array_equal(y, yr) and np.array_equal(oracle.max_pooling_backward(arg, dy, c, h, w, fh, fw, F), dxr)
        xb = synth.bernoulli_bits(rng, c * h * w, F, p=0.25)
        ybr, dxbr, _ = oracle.ref_max_pooling(xb, c, h, w, fh, fw, F, bit=True, dy=dy)
        assert np.array_equal(synth.unpack_bits(oracle.bit_max_pooling_forward(xb, c, h, w, fh, fw, F), F), synth.unpack_bits(ybr, F))
        assert np.array_equal(oracle.bit_max_pooling_backward(xb, dy, c, h, w, fh, fw, F), dxbr)
        for fill in (True, False):
            du = rng.standard_normal((c * h * fh * w * fw, F)).astype(F32)
            ur, dur, _ = oracle.ref_up_sampling(x, c, h, w, fh, fw, F, fill, dy=du)
            assert np.array_equal(oracle.up_sampling_forward(x, c, h, w, fh, fw, F, fill), ur)
            assert np.array_equal(oracle.up_sampling_backward(du, c, h, w, fh, fw, F, fill), dur)
            ubr, _, _ = oracle.ref_up_sampling(xb, c, h, w, fh, fw, F, fill, bit=True)
            assert np.array_equal(synth.unpack_bits(oracle.up_sampling_forward(xb, c, h, w, fh, fw, F, fill, bit=True), F), synth.unpack_bits(ubr, F))


def test_known_answers_of_the_reference_tests():
    # tests/gtest/MaxPoolingTest.cpp:9-146: 2 frames of 3 x 4 x 6 filled with 1000 f + 100 c + 10 y + x, one value raised to 99; 2 x 3 windows
    f, c, yy, xx = np.meshgrid(np.arange(2), np.arange(3), np.arange(4), np.arange(6), indexing="ij")
    img = (1000 * f + 100 * c + 10 * yy + xx).astype(F32)
    img[0, 0, 0, 1] = 99
    x = img.transpose(1, 2, 3, 0).reshape(3 * 4 * 6, 2)
    y, arg = oracle.max_pooling_forward(x, 3, 4, 6, 2, 3, 2)
    y4 = y.reshape(3, 2, 2, 2)                                          # [c, oy, ox, frame]
    assert [y4[0, 0, 0, 0], y4[0, 0, 1, 0], y4[0, 1, 0, 0], y4[0, 1, 1, 0]] == [99, 15, 32, 35]
    assert [y4[1, 0, 0, 0], y4[2, 1, 1, 0], y4[0, 0, 0, 1], y4[2, 1, 1, 1]] == [112, 235, 1012, 1235]
    f, c, yy, xx = np.meshgrid(np.arange(2), np.arange(3), np.arange(2), np.arange(2), indexing="ij")
    dy = (1000 * f + 100 * c + 10 * yy + xx + 1).astype(F32).transpose(1, 2, 3, 0).reshape(3 * 2 * 2, 2)
    dx = oracle.max_pooling_backward(arg, dy, 3, 4, 6, 2, 3, 2).reshape(3, 4, 6, 2)
    assert dx[0, 0, 1, 0] == 1 and dx[0, 1, 5, 0] == 2 and dx[0, 3, 2, 0] == 11 and dx[0, 0, 0, 0] == 0 and dx[0, 1, 2, 0] == 0
    assert np.count_nonzero(dx) == dy.size                              # one input per window and frame receives the gradient
    # tests/gtest/UpSamplingTest.cpp:21-120: 2 frames of 4 x 3 x 2, every pixel becomes a 2 x 3 block
    f, c, yy, xx = np.meshgrid(np.arange(2), np.arange(4), np.arange(3), np.arange(2), indexing="ij")
    x = (1000 * f + 100 * c + 10 * yy + xx).astype(F32).transpose(1, 2, 3, 0).reshape(4 * 3 * 2, 2)
    u = oracle.up_sampling_forward(x, 4, 3, 2, 2, 3, 2).reshape(4, 6, 6, 2)
    assert (u[0, 0:2, 0:3, 0] == 0).all() and (u[0, 0:2, 3:6, 0] == 1).all() and (u[0, 2:4, 3:6, 0] == 11).all()
    assert (u[1, 2:4, 3:6, 0] == 111).all() and (u[3, 4:6, 3:6, 1] == 1321).all()


def test_numpy_restatements():
    rng = np.random.default_rng(62)
    c, h, w, fh, fw, F = 3, 6, 8, 2, 4, 50                              # windows that divide the image: a reshape does the pooling
    x = rng.standard_normal((c * h * w, F)).astype(F32)
    y, arg = oracle.max_pooling_forward(x, c, h, w, fh, fw, F)
    win = x.reshape(c, h // fh, fh, w // fw, fw, F).transpose(0, 1, 3, 2, 4, 5).reshape(c, h // fh, w // fw, fh * fw, F)
    assert np.array_equal(y.reshape(c, h // fh, w // fw, F), win.max(axis=3))
    assert np.array_equal(arg.reshape(c, h // fh, w // fw, F), win.argmax(axis=3))
    dy = rng.standard_normal(y.shape).astype(F32)
    dx = oracle.max_pooling_backward(arg, dy, c, h, w, fh, fw, F)
    assert np.array_equal(dx.reshape(c, h // fh, fh, w // fw, fw, F).sum(axis=(2, 4)), dy.reshape(c, h // fh, w // fw, F))
    xb = synth.bernoulli_bits(rng, c * h * w, F, p=0.2)
    bits = synth.unpack_bits(xb, F).reshape(c, h // fh, fh, w // fw, fw, F)
    assert np.array_equal(synth.unpack_bits(oracle.bit_max_pooling_forward(xb, c, h, w, fh, fw, F), F).reshape(c, h // fh, w // fw, F),
                          bits.max(axis=(2, 4)))
    dxb = oracle.bit_max_pooling_backward(xb, dy, c, h, w, fh, fw, F).reshape(c, h // fh, fh, w // fw, fw, F)
    assert np.array_equal(dxb.sum(axis=(2, 4)), np.where(bits.max(axis=(2, 4)) > 0, dy.reshape(c, h // fh, w // fw, F), F32(0)))
    assert (dxb[bits == 0] == 0).all()
    # up-sampling is np.repeat; its backward with one channel of ones counts the block; pooling undoes a filled up-sampling
    u = oracle.up_sampling_forward(x, c, h, w, 2, 3, F)
    assert np.array_equal(u.reshape(c, h * 2, w * 3, F), np.repeat(np.repeat(x.reshape(c, h, w, F), 2, axis=1), 3, axis=2))
    assert np.array_equal(oracle.max_pooling_forward(u, c, h * 2, w * 3, 2, 3, F)[0], x)
    assert np.array_equal(oracle.up_sampling_backward(np.ones_like(u), c, h, w, 2, 3, F), np.full_like(x, 6))
    assert np.array_equal(oracle.up_sampling_backward(np.ones_like(u), c, h, w, 2, 3, F, fill=False), np.ones_like(x))
    sparse = oracle.up_sampling_forward(x, c, h, w, 2, 3, F, fill=False).reshape(c, h, 2, w, 3, F)
    assert np.array_equal(sparse[:, :, 1, :, 1, :], x.reshape(c, h, w, F)) and np.count_nonzero(sparse) == np.count_nonzero(x)
