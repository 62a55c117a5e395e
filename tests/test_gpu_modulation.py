"""GPU parity of RealToBinary, BinaryToReal, Binarize and HardTanh (through the C ABI) against the CPU oracle, bit for bit, and against
the vectors that the reference's own host classes wrote (tests/golden/modulation.npz): bit for bit where the layer is one comparison or
one division per element, and for RealToBinary on the cases whose arithmetic is exact; its other cases to the few units in the last
place by which the reference's build (fused multiply-adds) differs from the operation-by-operation arithmetic of oracle and kernels."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "modulation.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _odd(n):
    """a row pitch above n that is not a multiple of four floats: rows are not 16-byte aligned, the kernels go frame by frame"""
    return n + 1 if (n + 1) % 4 else n + 2


def _pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype)
    out[:, :a.shape[1]] = a
    return out


# depth, points, frames, frame modulation, depth modulation, lo, hi; strides aligned (wide accesses) or odd (frame by frame)
R2B_SHAPES = [(1, 784, 64, 7, 1, 0.0, 1.0), (3, 1024, 16, 15, 1, 0.0, 1.0), (2, 3, 33, 3, 4, -1.0, 2.0), (4, 2, 5, 15, 2, 0.1, 0.9),
              (3, 3, 40, 2, 3, 0.0, 255.0), (1, 1, 1, 1, 1, 0.0, 1.0), (1, 5, 3000, 1, 1, 0.0, 1.0), (2, 70000, 2, 3, 1, 0.0, 1.0),
              (1, 3, 100, 40, 1, 0.0, 1.0)]


@pytest.mark.parametrize("shape", R2B_SHAPES)
@pytest.mark.parametrize("aligned", [True, False])
def test_real_to_binary(ops, shape, aligned):
    d, p, F, fm, dm, lo, hi = shape
    rng = np.random.default_rng(int(sum(shape[:5])))
    yF = F * fm
    xs = synth.frame_stride_fp32(F) if aligned else _odd(F)
    ys = synth.frame_stride_fp32(yF) if aligned else _odd(yF)
    x = _pad((rng.random((d * p, F)) * (hi - lo) * 1.2 + lo - 0.1 * (hi - lo)).astype(F32), xs)
    x[0, 0] = np.nan
    for binarize in (True, False):
        want = oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=binarize, y_stride=ys)
        got = host(ops.real_to_binary_forward(dev(x), d, p, F, fm, dm, lo, hi, binarize=binarize, y_stride=ys))
        assert np.array_equal(got[:, :yF], want[:, :yF]), binarize
        ws = synth.frame_stride_bit(yF) if aligned else (yF + 31) // 32
        want = oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=binarize, bit=True, y_stride=ws)
        got = host(ops.real_to_binary_forward(dev(x), d, p, F, fm, dm, lo, hi, binarize=binarize, bit=True, y_stride=ws))
        assert np.array_equal(got, want), binarize          # whole rows: bits past the last frame and padding words are 0 on both sides


B2R_SHAPES = [(10, 10, 1024, 1), (70, 10, 1024, 7), (70, 10, 37, 7), (12, 3, 40, 15), (8, 8, 33, 3), (6, 1, 5, 2), (640, 10, 100, 33),
              (3, 3, 1, 1), (20, 10, 9, 64), (140000, 70000, 2, 3)]


@pytest.mark.parametrize("shape", B2R_SHAPES)
@pytest.mark.parametrize("aligned", [True, False])
def test_binary_to_real(ops, shape, aligned):
    I, O, Fy, fm = shape
    rng = np.random.default_rng(sum(shape))
    F = Fy * fm
    xs = synth.frame_stride_fp32(F) if aligned else _odd(F)
    ys = synth.frame_stride_fp32(Fy) if aligned else _odd(Fy)
    x = _pad(rng.standard_normal((I, F)).astype(F32), xs)
    x[:, F:] = 7.0                                      # padding must not be counted
    x[rng.random(x.shape) < 0.1] = 0.0
    y = host(ops.binary_to_real_forward(dev(x), O, Fy, fm, y_stride=ys))
    assert np.array_equal(y[:, :Fy], oracle.binary_to_real_forward(x, O, Fy, fm, y_stride=ys)[:, :Fy])
    ws = synth.frame_stride_bit(F) if aligned else (F + 31) // 32
    xb = synth.bernoulli_bits(rng, I, F, ws)
    if F % 32:                                          # set bits past the last frame must not be counted
        xb[:, F // 32] |= np.int32(-1) << (F % 32)
    xb[:, (F + 31) // 32:] = -1
    y = host(ops.binary_to_real_forward(dev(xb), O, Fy, fm, y_stride=ys))
    assert np.array_equal(y[:, :Fy], oracle.binary_to_real_forward(xb, O, Fy, fm, bit=True, y_stride=ys)[:, :Fy])
    dy = _pad(rng.standard_normal((O, Fy)).astype(F32), ys)
    dx = host(ops.binary_to_real_backward(dev(dy), I, Fy, fm, x_stride=xs))
    assert np.array_equal(dx[:, :F], oracle.binary_to_real_backward(dy, I, Fy, fm, x_stride=xs)[:, :F])


@pytest.mark.parametrize("shape", [(6144, 1024), (70, 37), (3, 1), (1, 5000), (70000, 3), (216, 230400 // 64)])
@pytest.mark.parametrize("aligned", [True, False])
def test_binarize_and_hard_tanh(ops, shape, aligned):
    nodes, F = shape
    rng = np.random.default_rng(nodes + F)
    stride = synth.frame_stride_fp32(F) if aligned else _odd(F)
    x = _pad(rng.standard_normal((nodes, F)).astype(F32), stride)
    dy = _pad(rng.standard_normal((nodes, F)).astype(F32), stride)
    lo, hi, th = F32(-0.7), F32(0.9), F32(0.1)
    x.flat[:7] = [lo, hi, th, 0.0, -0.0, np.nan, np.inf]
    assert np.array_equal(host(ops.binarize_forward(dev(x), F, th, -1.0, 1.0))[:, :F], oracle.binarize_forward(x, F, th, -1.0, 1.0)[:, :F])
    assert np.array_equal(host(ops.binarize_forward(dev(x), F, 0.0, 0.25, 0.75))[:, :F], oracle.binarize_forward(x, F, 0.0, 0.25, 0.75)[:, :F])
    ws = synth.frame_stride_bit(F) if aligned else (F + 31) // 32
    assert np.array_equal(host(ops.binarize_forward(dev(x), F, th, bit=True, y_stride=ws)), oracle.binarize_forward(x, F, th, bit=True, y_stride=ws))
    got, want = host(ops.hard_tanh_forward(dev(x), F, lo, hi))[:, :F], oracle.hard_tanh_forward(x, F, lo, hi)[:, :F]
    assert np.array_equal(got, want, equal_nan=True)
    assert np.array_equal(host(ops.hard_tanh_backward(dev(x), dev(dy), F, lo, hi))[:, :F], oracle.hard_tanh_backward(x, dy, F, lo, hi)[:, :F])


def test_reference_vectors(ops):
    for k in range(int(GOLD["r2b_count"][0])):
        q = "m%d_" % k
        d, p, F, fm, dm, dyadic = [int(v) for v in GOLD[q + "geom"]]
        lo, hi = [float(v) for v in GOLD[q + "range"]]
        x = dev(GOLD[q + "x"])
        yF = F * fm
        tol = 4e-7 * fm * dm * max(1.0, (abs(lo) + abs(hi)) / (hi - lo))
        real = host(ops.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=False))
        binary = host(ops.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=True))
        bits = synth.unpack_bits(host(ops.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=True, bit=True)), yF)
        near_half = np.abs(real - 0.5) <= tol
        for got, want in ((binary, GOLD[q + "y_binary"]), (bits, synth.unpack_bits(GOLD[q + "y_binary_bits"], yF))):
            bad = got != want
            assert not (bad & ~near_half).any() and not (dyadic and bad.any()), k
        if (q + "y_real") in GOLD:
            assert np.abs(real - GOLD[q + "y_real"]).max() <= tol and (not dyadic or np.array_equal(real, GOLD[q + "y_real"])), k
            real_bits = synth.unpack_bits(host(ops.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=False, bit=True)), yF)
            bad = real_bits != synth.unpack_bits(GOLD[q + "y_real_bits"], yF)
            assert not (bad & ~(real <= tol)).any() and not (dyadic and bad.any()), k
    for k in range(int(GOLD["b2r_count"][0])):
        q = "b%d_" % k
        I, O, Fy, fm = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(host(ops.binary_to_real_forward(dev(GOLD[q + "x"]), O, Fy, fm)), GOLD[q + "y"]), k
        assert np.array_equal(host(ops.binary_to_real_forward(dev(GOLD[q + "xbits"]), O, Fy, fm)), GOLD[q + "y_from_bits"]), k
        assert np.array_equal(host(ops.binary_to_real_backward(dev(GOLD[q + "dy"]), I, Fy, fm)), GOLD[q + "dx"]), k
    for k in range(int(GOLD["act_count"][0])):
        q = "a%d_" % k
        kind = bytes(GOLD[q + "kind"]).decode()
        nodes, F = [int(v) for v in GOLD[q + "geom"]]
        th, low, high, lo, hi = [F32(v) for v in GOLD[q + "params"]]
        x = dev(GOLD[q + "x"])
        if kind != "binarize":
            th = (lo + hi) / F32(2)
        if kind == "hard_tanh":
            assert np.array_equal(host(ops.hard_tanh_forward(x, F, lo, hi)), GOLD[q + "y"]), k
        else:
            assert np.array_equal(host(ops.binarize_forward(x, F, th, low, high)), GOLD[q + "y"]), k
        assert np.array_equal(host(ops.binarize_forward(x, F, th, bit=True)), GOLD[q + "y_bits"]), k
        assert np.array_equal(host(ops.hard_tanh_backward(x, dev(GOLD[q + "dy"]), F, lo, hi)), GOLD[q + "dx"]), k


def test_modulated_pipeline_round_trip(ops):
    """RealToBinary -> BinaryToReal with the same modulation size returns the input quantised to 1 / frames steps: the size-independent
    property of the pair, at a batch the oracle would take minutes for."""
    import torch
    rng = np.random.default_rng(77)
    nodes, F, fm = 784, 4096, 15
    x = rng.random((nodes, F)).astype(F32)
    bits = ops.real_to_binary_forward(dev(x), 1, nodes, F, frame_mod=fm, bit=True)
    y = host(ops.binary_to_real_forward(bits, nodes, F, fm))
    assert np.abs(y - x).max() <= 0.5 / fm + 1e-6
    real = ops.real_to_binary_forward(dev(x), 1, nodes, F, frame_mod=fm, binarize=True)
    assert np.array_equal(host(ops.binary_to_real_forward(real, nodes, F, fm)), y)
    assert np.array_equal(host(ops.binarize_forward(real, F * fm, 0.0, bit=True)), host(bits))
    torch.cuda.synchronize()


def test_bad_arguments(ops):
    from binarybrain_amd.capi import BbhipError
    x = dev(np.zeros((4, 64), F32))
    with pytest.raises(BbhipError):
        ops.binary_to_real_forward(x, 2, 32, 4)             # 128 input frames in rows of 64
    with pytest.raises(BbhipError):
        ops.real_to_binary_forward(x, 1, 4, 64, frame_mod=0)
    with pytest.raises(BbhipError):
        ops.hard_tanh_forward(x, 65)
