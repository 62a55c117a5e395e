"""The oracle's RealToBinary, BinaryToReal, Binarize and HardTanh, pinned without a GPU: vectors written by the reference's own host
classes (tests/golden/modulation.npz), the compiled reference where oracle/_ref is present, the known answers of the reference's tests
(tests/gtest/RealToBinaryTest.cpp:42-180, BinaryToRealTest.cpp, BinarizeTest.cpp) and numpy restatements.

BinaryToReal, Binarize and HardTanh are one comparison or one division per element: bit-exact.  RealToBinary is three
subtract-and-scale steps; the reference's build fuses some of its multiply-add pairs (which ones is the compiler's choice), the oracle
rounds every operation: on inputs where every operation is exact ("dyadic" cases) the two agree bit for bit, elsewhere to a few units
in the last place times the modulation sizes, and binarized outputs may differ only where the value sits that close to the threshold."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "modulation.npz"))
F32 = np.float32


def real_to_binary_fp64(x, d, p, F, fm, dm, lo, hi):
    """the layer's value before binarization, in float64: [d * dm * p, F * fm]"""
    v = (x.astype(np.float64).reshape(d, 1, p, F, 1) - lo) / (hi - lo)
    v = (v - np.arange(dm).reshape(1, dm, 1, 1, 1) / dm) * dm
    v = (v - np.arange(fm).reshape(1, 1, 1, 1, fm) / fm) * fm
    return np.clip(v, 0.0, 1.0).reshape(d * dm * p, F * fm)


def check_real_to_binary(x, d, p, F, fm, dm, lo, hi, want_binary, want_bits, want_real, want_real_bits, exact):
    ref64 = real_to_binary_fp64(x, d, p, F, fm, dm, lo, hi)
    tol = 4e-7 * fm * dm * max(1.0, (abs(lo) + abs(hi)) / (hi - lo))
    real = oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=False)
    assert np.abs(real - ref64).max() <= tol
    binary = oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=True)
    bits = synth.unpack_bits(oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=True, bit=True), F * fm)
    real_bits = synth.unpack_bits(oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=False, bit=True), F * fm)
    assert np.array_equal(binary, np.where(real > 0.5, F32(1), F32(-1)))
    assert np.array_equal(bits, real > 0.5) and np.array_equal(real_bits, real > 0)
    if exact:
        assert np.array_equal(real, ref64.astype(F32))
    near_half = np.abs(ref64 - 0.5) <= tol
    near_zero = (ref64 <= tol)
    if want_binary is not None:
        bad = binary != want_binary
        assert not (bad & ~near_half).any() and (not exact or not bad.any())
        bad = bits != synth.unpack_bits(want_bits, F * fm)
        assert not (bad & ~near_half).any() and (not exact or not bad.any())
    if want_real is not None:
        assert np.abs(real - want_real).max() <= tol and (not exact or np.array_equal(real, want_real))
        bad = real_bits != synth.unpack_bits(want_real_bits, F * fm)
        assert not (bad & ~near_zero).any() and (not exact or not bad.any())


def test_reference_vectors_real_to_binary():
    for k in range(int(GOLD["r2b_count"][0])):
        q = "m%d_" % k
        d, p, F, fm, dm, dyadic = [int(v) for v in GOLD[q + "geom"]]
        lo, hi = [float(v) for v in GOLD[q + "range"]]
        have_real = (q + "y_real") in GOLD
        check_real_to_binary(GOLD[q + "x"], d, p, F, fm, dm, lo, hi, GOLD[q + "y_binary"], GOLD[q + "y_binary_bits"],
                             GOLD[q + "y_real"] if have_real else None, GOLD[q + "y_real_bits"] if have_real else None, bool(dyadic))


def test_reference_vectors_binary_to_real_and_activations():
    for k in range(int(GOLD["b2r_count"][0])):
        q = "b%d_" % k
        I, O, Fy, fm = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(oracle.binary_to_real_forward(GOLD[q + "x"], O, Fy, fm), GOLD[q + "y"]), k
        assert np.array_equal(oracle.binary_to_real_forward(GOLD[q + "xbits"], O, Fy, fm, bit=True), GOLD[q + "y_from_bits"]), k
        assert np.array_equal(oracle.binary_to_real_backward(GOLD[q + "dy"], I, Fy, fm), GOLD[q + "dx"]), k
    for k in range(int(GOLD["act_count"][0])):
        q = "a%d_" % k
        kind = bytes(GOLD[q + "kind"]).decode()
        nodes, F = [int(v) for v in GOLD[q + "geom"]]
        th, low, high, lo, hi = [F32(v) for v in GOLD[q + "params"]]
        x = GOLD[q + "x"]
        if kind != "binarize":
            th = (lo + hi) / F32(2)                     # HardTanh's threshold, include/bb/HardTanh.h:70
        if kind == "hard_tanh":
            assert np.array_equal(oracle.hard_tanh_forward(x, F, lo, hi), GOLD[q + "y"]), k
        else:
            assert np.array_equal(oracle.binarize_forward(x, F, th, low, high), GOLD[q + "y"]), k
        assert np.array_equal(oracle.binarize_forward(x, F, th, bit=True), GOLD[q + "y_bits"]), k
        assert np.array_equal(oracle.hard_tanh_backward(x, GOLD[q + "dy"], F, lo, hi), GOLD[q + "dx"]), k


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_against_compiled_reference():
    rng = np.random.default_rng(51)
    for (d, p, F, fm, dm, lo, hi, dyadic) in [(3, 7, 21, 7, 1, 0.0, 1.0, False), (2, 5, 40, 3, 5, -2.0, 3.0, False), (1, 9, 70, 16, 2, 0.0, 1.0, True),
                                              (5, 1, 3, 1, 1, 0.0, 1.0, False), (2, 2, 64, 15, 3, 0.0, 255.0, False)]:
        if dyadic:
            x = (rng.integers(-8, 265, (d * p, F)) / 256.0).astype(F32)
        else:
            x = (rng.random((d * p, F)) * (hi - lo) * 1.2 + lo - 0.1 * (hi - lo)).astype(F32)
        yb, _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, True)
        ybits, _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, True, bit=True)
        yr = yrbits = None
        if dm > 1:
            yr, _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, False)
            yrbits, _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, False, bit=True)
        check_real_to_binary(x, d, p, F, fm, dm, lo, hi, yb, ybits, yr, yrbits, dyadic)
    for bit in (False, True):
        for (I, O, Fy, fm) in [(30, 10, 12, 5), (9, 9, 40, 1), (64, 2, 7, 15), (5, 5, 3, 4)]:
            F = Fy * fm
            x = synth.bernoulli_bits(rng, I, F) if bit else rng.standard_normal((I, F)).astype(F32)
            dy = rng.standard_normal((O, Fy)).astype(F32)
            y, dx, _ = oracle.ref_binary_to_real(x, O, F, fm, bit=bit, dy=dy)
            assert np.array_equal(oracle.binary_to_real_forward(x, O, Fy, fm, bit=bit), y)
            assert np.array_equal(oracle.binary_to_real_backward(dy, I, Fy, fm), dx)
    for kind in ("binarize", "hard_tanh", "hard_tanh_binary"):
        for bit in (False, True):
            nodes, F = 6, 77
            x = rng.standard_normal((nodes, F)).astype(F32); dy = rng.standard_normal((nodes, F)).astype(F32)
            th, low, high, lo, hi = F32(0.2), F32(-1), F32(1), F32(-0.6), F32(0.8)
            y, dx, _ = oracle.ref_activation(kind, x, F, bit=bit, th=th, low=low, high=high, lo=lo, hi=hi, dy=dy)
            t = th if kind == "binarize" else (lo + hi) / F32(2)
            if kind == "hard_tanh" and not bit:
                got = oracle.hard_tanh_forward(x, F, lo, hi)
            else:
                got = oracle.binarize_forward(x, F, t, low, high, bit=bit)
            if bit:
                got, y = synth.unpack_bits(got, F), synth.unpack_bits(y, F)
            assert np.array_equal(got, y), (kind, bit)
            assert np.array_equal(oracle.hard_tanh_backward(x, dy, F, lo, hi), dx), (kind, bit)


def test_known_answers_of_the_reference_tests():
    # tests/gtest/RealToBinaryTest.cpp:42-180: shape {2, 3}, frame modulation 2, depth modulation 3, one frame
    x = np.array([[0.1], [0.2], [0.5], [1.0], [0.0], [0.9]], F32)
    real = oracle.real_to_binary_forward(x, 2, 3, 1, frame_mod=2, depth_mod=3, binarize=False).reshape(6, 3, 2)       # [depth, point, frame]
    want = np.zeros((6, 3, 2))
    want[0, 0] = [0.6, 0.0]; want[0, 1] = [1.0, 0.2]; want[0, 2] = [1.0, 1.0]; want[1, 2] = [1.0, 0.0]
    want[3:6, 0] = 1.0; want[3:6, 2] = 1.0; want[5, 2] = [1.0, 0.4]
    assert np.abs(real - want).max() < 1e-6
    binary = oracle.real_to_binary_forward(x, 2, 3, 1, frame_mod=2, depth_mod=3, binarize=True).reshape(6, 3, 2)
    assert np.array_equal(binary, np.where(want > 0.5, 1.0, -1.0))
    # :186-215: three nodes, modulation 2, packed output: 0.0 -> clear, 1.0 -> set in both frames
    bits = synth.unpack_bits(oracle.real_to_binary_forward(np.array([[0.0], [1.0], [0.5]], F32), 3, 1, 1, frame_mod=2, bit=True), 2)
    assert np.array_equal(bits[0], [0, 0]) and np.array_equal(bits[1], [1, 1])
    # tests/gtest/BinaryToRealTest.cpp:9-121 (disabled in the reference, the numbers still hold): three nodes, two frames fold into one
    x = np.array([[1, 1], [0, 0], [0, 1]], F32)
    assert np.array_equal(oracle.binary_to_real_forward(x, 3, 1, 2), np.array([[1.0], [0.0], [0.5]], F32))
    assert np.array_equal(oracle.binary_to_real_forward(synth.pack_bits(x.astype(np.uint8)), 3, 1, 2, bit=True), np.array([[1.0], [0.0], [0.5]], F32))
    # its backward numbers (dx = dy in both frames) come from a version without the 1 / frames gain; today's host loop halves them
    assert np.array_equal(oracle.binary_to_real_backward(np.array([[0.0], [1.0], [0.5]], F32), 3, 1, 2), np.array([[0, 0], [0.5, 0.5], [0.25, 0.25]], F32))
    # tests/gtest/BinarizeTest.cpp:9-50: sign with the threshold at 0, gradient passed inside (-1, 1); nodes x frames below
    x = np.array([[-1.01, -0.1], [-0.9, 0.9], [-0.5, 1.01]], F32)
    assert np.array_equal(oracle.binarize_forward(x, 2), np.array([[-1, -1], [-1, 1], [-1, 1]], F32))
    dy = np.array([[1, 4], [2, 5], [3, 6]], F32)
    assert np.array_equal(oracle.hard_tanh_backward(x, dy, 2), np.array([[0, 4], [2, 5], [3, 0]], F32))
    # :53-99, packed output
    x = np.array([[-1.01, 0.99, -0.5], [-0.99, 0.01, 1.01]], F32)
    assert np.array_equal(synth.unpack_bits(oracle.binarize_forward(x, 3, bit=True), 3), np.array([[0, 1, 0], [0, 1, 1]]))
    assert np.array_equal(oracle.hard_tanh_backward(x, np.array([[1, 2, 3], [4, 5, 6]], F32), 3), np.array([[0, 2, 3], [4, 5, 0]], F32))


def test_numpy_restatements():
    rng = np.random.default_rng(52)
    I, O, Fy, fm = 42, 6, 25, 7
    x = rng.standard_normal((I, Fy * fm)).astype(F32)
    y = oracle.binary_to_real_forward(x, O, Fy, fm)
    share = (x > 0).reshape(I // O, O, Fy, fm).sum(axis=(0, 3)).astype(F32) / F32(I // O * fm)
    assert np.array_equal(y, share)
    xb = synth.pack_bits((x > 0).astype(np.uint8))
    assert np.array_equal(oracle.binary_to_real_forward(xb, O, Fy, fm, bit=True), share)
    dy = rng.standard_normal((O, Fy)).astype(F32)
    dx = oracle.binary_to_real_backward(dy, I, Fy, fm)
    gain = F32(O) / (F32(I) * F32(fm))
    assert np.array_equal(dx, np.tile(np.repeat(dy * gain, fm, axis=1), (I // O, 1)))
    # forward of ones is 1, the backward spreads a gradient whose sum over a fold is dy * O * ... / I: total preserved up to the gain
    assert np.abs(dx.astype(np.float64).reshape(I // O, O, Fy, fm).sum(axis=(0, 3)) - dy).max() < 1e-5
    v = rng.standard_normal((4, 50)).astype(F32) * 2
    lo, hi = F32(-0.75), F32(1.25)
    assert np.array_equal(oracle.hard_tanh_forward(v, 50, lo, hi), np.clip(v, lo, hi))
    g = rng.standard_normal((4, 50)).astype(F32)
    assert np.array_equal(oracle.hard_tanh_backward(v, g, 50, lo, hi), np.where((v > lo) & (v < hi), g, F32(0)))
    assert np.array_equal(oracle.binarize_forward(v, 50, 0.3, 0.0, 1.0), (v > F32(0.3)).astype(F32))
    assert np.array_equal(synth.unpack_bits(oracle.binarize_forward(v, 50, 0.3, bit=True), 50), v > F32(0.3))
    # NaN: comparisons are false — Binarize gives `low`, HardTanh passes the NaN and its gradient; RealToBinary's min/max turn it into 1
    n = np.array([[np.nan, 0.25]], F32)
    assert np.array_equal(oracle.binarize_forward(n, 2), np.array([[-1, 1]], F32))
    assert np.isnan(oracle.hard_tanh_forward(n, 2)[0, 0]) and oracle.hard_tanh_backward(n, np.array([[3, 4]], F32), 2)[0, 0] == 3
    assert oracle.real_to_binary_forward(n, 1, 1, 2, binarize=False)[0, 0] == 1.0
    # frame modulation sweeps the threshold: the share of set frames approximates the input
    x = rng.random((5, 8)).astype(F32)
    fm = 32
    bits = synth.unpack_bits(oracle.real_to_binary_forward(x, 5, 1, 8, frame_mod=fm, bit=True), 8 * fm)
    assert np.abs(bits.reshape(5, 8, fm).mean(axis=2) - x).max() <= 0.5 / fm + 1e-6
