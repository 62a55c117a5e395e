"""GPU parity of Shuffle (through the C ABI), fp32 rows and packed rows, against the CPU oracle and against the vectors that the
reference's own host class wrote (tests/golden/pooling.npz, keys s*): a permutation of whole rows, bit for bit."""
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


# nodes, shuffle unit, frames
SHAPES = [(6, 3, 2), (84, 7, 33), (64, 1, 5), (64, 64, 40), (30, 5, 70), (1024, 32, 1000), (36 * 900, 36, 256), (4096, 64, 8192), (1, 1, 1),
          (210, 14, 129)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("aligned", [True, False])
def test_shuffle(ops, shape, aligned):
    nodes, unit, F = shape
    rng = np.random.default_rng(sum(shape))
    stride = synth.frame_stride_fp32(F) if aligned else (F + 1 if (F + 1) % 4 else F + 2)
    x = rng.standard_normal((nodes, stride)).astype(F32)                # rows move whole: the padding travels with them
    x.flat[:3] = [np.nan, -np.inf, np.inf]
    y = host(ops.shuffle_forward(dev(x), unit, F))
    assert np.array_equal(y.view(np.int32), oracle.shuffle_forward(x, unit).view(np.int32))
    dx = host(ops.shuffle_backward(dev(x), unit, F))
    assert np.array_equal(dx.view(np.int32), oracle.shuffle_backward(x, unit).view(np.int32))
    ws = synth.frame_stride_bit(F) if aligned else (F + 31) // 32
    xb = synth.bernoulli_bits(rng, nodes, F, ws)
    assert np.array_equal(host(ops.shuffle_forward(dev(xb), unit, F)), oracle.shuffle_forward(xb, unit))
    assert np.array_equal(host(ops.shuffle_backward(dev(xb), unit, F)), oracle.shuffle_backward(xb, unit))


def test_views_that_are_not_16_byte_aligned(ops):
    import torch
    rng = np.random.default_rng(5)
    nodes, unit, stride = 40, 8, 64
    flat = dev(rng.standard_normal(nodes * stride + 1).astype(F32))
    x = flat[1:].view(nodes, stride)                                    # 4-byte aligned only: word by word
    want = oracle.shuffle_forward(host(x), unit)
    assert np.array_equal(host(ops.shuffle_forward(x, unit, stride)), want)
    out = torch.empty(nodes * stride + 1, dtype=torch.float32, device=flat.device)[1:].view(nodes, stride)
    from binarybrain_amd import capi
    from binarybrain_amd.ops import check, ptr, stream_ptr
    check(capi.lib().bbhip_Shuffle_Forward(ptr(flat[:-1].view(nodes, stride)), ptr(out), unit, nodes, stride, stride, stream_ptr()))
    assert np.array_equal(host(out), oracle.shuffle_forward(host(flat[:-1].view(nodes, stride)), unit))


def test_reference_vectors(ops):
    for k in range(int(GOLD["shuffle_count"][0])):
        q = "s%d_" % k
        nodes, unit, F = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(host(ops.shuffle_forward(dev(GOLD[q + "x"]), unit, F)), GOLD[q + "y"]), k
        assert np.array_equal(host(ops.shuffle_backward(dev(GOLD[q + "dy"]), unit, F)), GOLD[q + "dx"]), k
        assert np.array_equal(host(ops.shuffle_forward(dev(GOLD[q + "xbits"]), unit, F)), GOLD[q + "y_bits"]), k
        assert np.array_equal(host(ops.shuffle_backward(dev(GOLD[q + "dybits"]), unit, F)), GOLD[q + "dx_bits"]), k


def test_round_trip_at_full_size(ops):
    import torch
    nodes, unit, F = 8192, 128, 8192                                    # 256 MiB of fp32 rows
    x = torch.randn((nodes, F), device="cuda")
    y = ops.shuffle_forward(x, unit, F)
    assert torch.equal(y, x.view(unit, nodes // unit, F).transpose(0, 1).reshape(nodes, F))
    assert torch.equal(ops.shuffle_backward(y, unit, F), x)


def test_refusals(ops):
    from binarybrain_amd import capi
    x = dev(np.zeros((6, 4), F32))
    with pytest.raises(capi.BbhipError, match="multiple of the unit size"):
        ops.shuffle_forward(x, 4, 4)
    with pytest.raises(capi.BbhipError, match="multiple of the unit size"):
        ops.shuffle_backward(x, 4, 4)
    with pytest.raises(capi.BbhipError, match="positive"):
        ops.shuffle_forward(x, 0, 4)
