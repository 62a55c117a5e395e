"""GPU parity of MaxPooling and UpSampling (through the C ABI), fp32 and packed bits, against the CPU oracle and against the vectors
that the reference's own host classes wrote (tests/golden/pooling.npz): selections and sums in a fixed order, bit for bit."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "pooling.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _odd(n):
    """a row pitch above n that is not a multiple of four floats: the kernels go frame by frame"""
    return n + 1 if (n + 1) % 4 else n + 2


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


# channels, height, width, filter height, filter width, frames
POOL_SHAPES = [(36, 30, 30, 2, 2, 256), (3, 4, 6, 2, 3, 2), (2, 5, 7, 2, 2, 33), (1, 8, 8, 3, 3, 64), (4, 3, 3, 1, 1, 5), (2, 6, 5, 2, 4, 40),
               (2, 7, 7, 7, 7, 100), (1, 1, 1, 2, 2, 1), (3, 9, 4, 1, 5, 70), (64, 16, 16, 2, 2, 1000)]


@pytest.mark.parametrize("shape", POOL_SHAPES)
@pytest.mark.parametrize("aligned", [True, False])
def test_max_pooling(ops, shape, aligned):
    c, h, w, fh, fw, F = shape
    rng = np.random.default_rng(sum(shape))
    stride = synth.frame_stride_fp32(F) if aligned else _odd(F)
    x = _pad(rng.standard_normal((c * h * w, F)).astype(F32), stride)
    x[rng.random(x.shape) < 0.2] = 0.5                                  # ties: the first largest value wins
    x.flat[:3] = [np.nan, -np.inf, np.inf]
    O = c * ((h + fh - 1) // fh) * ((w + fw - 1) // fw)
    dy = _pad(rng.standard_normal((O, F)).astype(F32), stride)
    y, arg = ops.max_pooling_forward(dev(x), c, h, w, fh, fw, F)
    y_ref, arg_ref = oracle.max_pooling_forward(x, c, h, w, fh, fw, F)
    assert np.array_equal(host(y)[:, :F], y_ref[:, :F]) and np.array_equal(host(arg)[:, :F], arg_ref[:, :F])
    dx = host(ops.max_pooling_backward(arg, dev(dy), c, h, w, fh, fw, F))
    assert np.array_equal(dx[:, :F], oracle.max_pooling_backward(arg_ref, dy, c, h, w, fh, fw, F)[:, :F])
    ws = synth.frame_stride_bit(F) if aligned else (F + 31) // 32
    xb = synth.bernoulli_bits(rng, c * h * w, F, ws, p=0.3)
    assert np.array_equal(host(ops.bit_max_pooling_forward(dev(xb), c, h, w, fh, fw, F))[:, :(F + 31) // 32],
                          oracle.bit_max_pooling_forward(xb, c, h, w, fh, fw, F)[:, :(F + 31) // 32])
    dxb = host(ops.bit_max_pooling_backward(dev(xb), dev(dy), c, h, w, fh, fw, F))
    assert np.array_equal(dxb[:, :F], oracle.bit_max_pooling_backward(xb, dy, c, h, w, fh, fw, F)[:, :F])


# channels, height, width, filter height, filter width, frames
UP_SHAPES = [(36, 15, 15, 2, 2, 256), (3, 2, 3, 2, 2, 7), (2, 4, 3, 3, 2, 33), (1, 5, 5, 1, 1, 64), (4, 3, 2, 2, 3, 40), (2, 3, 3, 4, 5, 100)]


@pytest.mark.parametrize("shape", UP_SHAPES)
@pytest.mark.parametrize("fill", [True, False])
@pytest.mark.parametrize("aligned", [True, False])
def test_up_sampling(ops, shape, fill, aligned):
    c, h, w, fh, fw, F = shape
    rng = np.random.default_rng(sum(shape) + int(fill))
    stride = synth.frame_stride_fp32(F) if aligned else _odd(F)
    x = _pad(rng.standard_normal((c * h * w, F)).astype(F32), stride)
    dy = _pad(rng.standard_normal((c * h * fh * w * fw, F)).astype(F32), stride)
    assert np.array_equal(host(ops.up_sampling_forward(dev(x), c, h, w, fh, fw, F, fill))[:, :F], oracle.up_sampling_forward(x, c, h, w, fh, fw, F, fill)[:, :F])
    assert np.array_equal(host(ops.up_sampling_backward(dev(dy), c, h, w, fh, fw, F, fill))[:, :F], oracle.up_sampling_backward(dy, c, h, w, fh, fw, F, fill)[:, :F])
    ws = synth.frame_stride_bit(F) if aligned else (F + 31) // 32
    xb = synth.bernoulli_bits(rng, c * h * w, F, ws)
    assert np.array_equal(host(ops.up_sampling_forward(dev(xb), c, h, w, fh, fw, F, fill))[:, :(F + 31) // 32],
                          oracle.up_sampling_forward(xb, c, h, w, fh, fw, F, fill, bit=True)[:, :(F + 31) // 32])


def test_reference_vectors(ops):
    for k in range(int(GOLD["pool_count"][0])):
        q = "p%d_" % k
        c, h, w, fh, fw, F = [int(v) for v in GOLD[q + "geom"]]
        y, arg = ops.max_pooling_forward(dev(GOLD[q + "x"]), c, h, w, fh, fw, F)
        assert np.array_equal(host(y), GOLD[q + "y"]), k
        assert np.array_equal(host(ops.max_pooling_backward(arg, dev(GOLD[q + "dy"]), c, h, w, fh, fw, F)), GOLD[q + "dx"]), k
        xb = dev(GOLD[q + "xbits"])
        assert np.array_equal(host(ops.bit_max_pooling_forward(xb, c, h, w, fh, fw, F)), GOLD[q + "y_bits"]), k
        assert np.array_equal(host(ops.bit_max_pooling_backward(xb, dev(GOLD[q + "dy"]), c, h, w, fh, fw, F)), GOLD[q + "dx_from_bits"]), k
    for k in range(int(GOLD["up_count"][0])):
        q = "u%d_" % k
        c, h, w, fh, fw, fill, F = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(host(ops.up_sampling_forward(dev(GOLD[q + "x"]), c, h, w, fh, fw, F, bool(fill))), GOLD[q + "y"]), k
        assert np.array_equal(host(ops.up_sampling_backward(dev(GOLD[q + "dy"]), c, h, w, fh, fw, F, bool(fill))), GOLD[q + "dx"]), k
        assert np.array_equal(host(ops.up_sampling_forward(dev(GOLD[q + "xbits"]), c, h, w, fh, fw, F, bool(fill))), GOLD[q + "y_bits"]), k


def test_pooling_undoes_up_sampling_at_full_size(ops):
    """size-independent properties at a batch the oracle would take long for: MaxPooling(UpSampling(x)) = x, the pooled gradient reaches
    one input per window, and the packed forms agree with the fp32 forms on 0 / 1 images"""
    import torch
    c, h, w, F = 64, 16, 16, 4096
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    x = torch.rand((c * h * w, F), device="cuda", generator=g)
    up = ops.up_sampling_forward(x, c, h, w, 2, 2, F)
    y, arg = ops.max_pooling_forward(up, c, 2 * h, 2 * w, 2, 2, F)
    assert torch.equal(y, x) and int(arg.max()) == 0                    # four equal values: the first wins
    dy = torch.randn((c * h * w, F), device="cuda", generator=g)
    dx = ops.max_pooling_backward(arg, dy, c, 2 * h, 2 * w, 2, 2, F)
    assert torch.equal(ops.up_sampling_backward(dx, c, h, w, 2, 2, F), dy)      # three zeros and dy, summed
    bits = (x > 0.7)
    packed = ops.binarize_forward(x, F, 0.7, bit=True)
    pooled = ops.bit_max_pooling_forward(packed, c, h, w, 2, 2, F)
    ref, _ = ops.max_pooling_forward(bits.float(), c, h, w, 2, 2, F)
    assert torch.equal(pooled, ops.binarize_forward(ref, F, 0.5, bit=True))


def test_bad_arguments(ops):
    from binarybrain_amd.capi import BbhipError, lib, check
    from binarybrain_amd.ops import ptr
    x = dev(np.zeros((2 * 4 * 4, 64), F32))
    y = dev(np.zeros((2 * 2 * 2, 64), F32)); arg = dev(np.zeros((2 * 2 * 2, 64), np.int32))
    with pytest.raises(BbhipError):                                     # output size that is not ceil(input / filter)
        check(lib().bbhip_fp32_MaxPooling_Forward(ptr(x), ptr(y), ptr(arg), 2, 2, 4, 4, 3, 2, 2, 64, 64, None))
    with pytest.raises(BbhipError):
        ops.up_sampling_forward(x, 2, 4, 4, 0, 2, 64)
    with pytest.raises(BbhipError):
        ops.max_pooling_forward(x, 2, 4, 4, 2, 2, 65)
