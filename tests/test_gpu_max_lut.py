"""GPU parity of MaxLut (through the C ABI) against the CPU oracle and against the vectors that the reference's own host class
wrote (tests/golden/maxlut.npz).  Maxima, ORs and gradients routed in table order: bit-exact."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "maxlut.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


SHAPES = [
    # n, I, O, frames
    (6, 12, 2, 3),              # the reference's own test
    (6, 70, 10, 1024),
    (4, 9, 5, 64),
    (1, 3, 3, 5),
    (8, 8, 2, 100),             # every node sees every input
    (15, 200, 33, 300),
    (300, 40, 3, 70),           # far more connections than inputs: every input repeats inside a node
    (6, 6144, 1024, 130),
    (4, 3136, 784, 257),        # 2 x 2 pooling over 28 x 28 x 4 as a wired layer
]


@pytest.mark.parametrize("shape", SHAPES)
def test_forward_and_backward(ops, shape):
    n, I, O, F = shape
    rng = np.random.default_rng(sum(shape))
    idx = rng.integers(0, I, (O, n)).astype(np.int32)
    stride = synth.frame_stride_fp32(F)
    x = (rng.random((I, F)) * 3 - 2).astype(F32)                # in [-2, 1): some nodes see nothing above the floor of -1
    x[rng.random(x.shape) < 0.1] = 0.0
    x[:, ::7] = np.round(x[:, ::7])                              # ties between inputs
    x = _pad(x, stride)
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    for bin_in in (False, True):
        for bin_out in (False, True):
            y = host(ops.max_lut_forward(dev(x), dev(idx), F, bin_in, bin_out))
            assert np.array_equal(y[:, :F], oracle.max_lut_forward(x, idx, F, bin_in, bin_out)[:, :F]), (bin_in, bin_out)
        dx = host(ops.max_lut_backward(dev(x), dev(dy), dev(idx), F, bin_in))
        want = oracle.max_lut_backward(x, dy, idx, F, bin_in)
        assert np.array_equal(dx[:, :F], want[:, :F]), bin_in
        assert np.all(dx[:, F:] == 0.0)
    sw = synth.frame_stride_bit(F)
    xb = synth.bernoulli_bits(rng, I, F, sw, p=0.15)
    yb = host(ops.bit_max_lut_forward(dev(xb), dev(idx), F))
    assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(oracle.bit_max_lut_forward(xb, idx, F), F))
    dxb = host(ops.bit_max_lut_backward(dev(xb), dev(dy), dev(idx), F))
    assert np.array_equal(dxb[:, :F], oracle.bit_max_lut_backward(xb, dy, idx, F)[:, :F])
    # every node hands its dy to exactly one input: the columns of dx and dy add up to the same, to the rounding of the sums
    assert np.allclose(dxb[:, :F].astype(np.float64).sum(axis=0), dy[:, :F].astype(np.float64).sum(axis=0), atol=1e-3)


def test_reference_vectors(ops):
    for k in range(int(GOLD["count"][0])):
        p = "m%d_" % k
        n, I, O, F, bin_out = [int(v) for v in GOLD[p + "geom"]]
        idx = GOLD[p + "idx"]
        stride = synth.frame_stride_fp32(F)
        x = _pad(GOLD[p + "x"], stride); dy = _pad(GOLD[p + "dy"], stride)
        assert np.array_equal(host(ops.max_lut_forward(dev(x), dev(idx), F, False, bool(bin_out)))[:, :F], GOLD[p + "y"]), k
        assert np.array_equal(host(ops.max_lut_backward(dev(x), dev(dy), dev(idx), F))[:, :F], GOLD[p + "dx"]), k
        xb = _pad(GOLD[p + "xbits"], synth.frame_stride_bit(F))
        yb = host(ops.bit_max_lut_forward(dev(xb), dev(idx), F))
        assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(GOLD[p + "ybits"], F)), k
        assert np.array_equal(host(ops.bit_max_lut_backward(dev(xb), dev(dy), dev(idx), F))[:, :F], GOLD[p + "dxbits"]), k


def test_bits_agree_with_the_fp32_path_on_plus_minus_one(ops):
    rng = np.random.default_rng(8)
    n, I, O, F = 6, 100, 64, 200
    idx = rng.integers(0, I, (O, n)).astype(np.int32)
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F), p=0.2)
    stride = synth.frame_stride_fp32(F)
    xf = _pad(synth.unpack_bits(xb, F).astype(F32) * 2 - 1, stride)
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    yb = synth.unpack_bits(host(ops.bit_max_lut_forward(dev(xb), dev(idx), F)), F)
    yf = host(ops.max_lut_forward(dev(xf), dev(idx), F))[:, :F]
    assert np.array_equal(yb.astype(F32) * 2 - 1, yf)
    assert np.array_equal(host(ops.bit_max_lut_backward(dev(xb), dev(dy), dev(idx), F))[:, :F],
                          host(ops.max_lut_backward(dev(xf), dev(dy), dev(idx), F))[:, :F])


def test_rejected_arguments(ops):
    import torch
    from binarybrain_amd import capi
    x = torch.zeros((4, 64), dtype=torch.float32, device="cuda")
    idx = torch.zeros((2, 3), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.BbhipError):
        ops.max_lut_forward(x, idx, 65)
    with pytest.raises(capi.BbhipError):
        ops.max_lut_forward(x, idx, 0)
    with pytest.raises(capi.BbhipError):
        ops.max_lut_backward(x, torch.zeros((2, 128), dtype=torch.float32, device="cuda"), idx, 64)
