"""CPU suite: pins the oracle (oracle/bb_oracle.c) before anything is compared against it.

Three independent anchors:
  1. vectors written by the reference's own CPU headers (tests/golden/*.npz, made by tests/golden/make_golden.py);
  2. the real reference compiled in place (oracle/_ref/libbbref.so) on fresh random inputs, where that library exists;
  3. what the mathematics fixes: corner inputs select table entries, constant tables, sum rules, multilinear finite
     differences, an fp64 brute force, BinaryLut6 == StochasticLut on {0,1} data, batch-norm gradient invariants.
"""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rel(a, b):
    return float(np.abs(a.astype(np.float64) - b).max() / max(1e-30, np.abs(b).max()))


# ------------------------------------------------------------------ 1. golden vectors

def test_golden_stochastic_lut():
    g = np.load(os.path.join(GOLD, "stochastic_lut.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        n, I, O, F, simd, binary_mode, lut_binarize = [int(v) for v in g[p + "meta"]]
        Wc = oracle.vector_clamp(g[p + "W"])
        assert np.array_equal(Wc, g[p + "Wc"])
        if simd >= 0:
            y = oracle.stochastic_lut_forward(n, g[p + "x"], g[p + "idx"], Wc, F, binary_mode, lut_binarize, 0.25, simd)
            dx, dW = oracle.stochastic_lut_backward(n, g[p + "x"], g[p + "dy"], g[p + "idx"], Wc, F, g[p + "dW0"],
                                                    binary_mode, lut_binarize, 0.25, simd)
        else:
            y = oracle.bit_stochastic_lut_forward(n, g[p + "xbits"], g[p + "idx"], Wc, F, F, lut_binarize)
            dx, dW = oracle.bit_stochastic_lut_backward(n, g[p + "xbits"], g[p + "dy"], g[p + "idx"], Wc, F, None, lut_binarize)
        if n >= 3:      # same association, same rounding: identical bits
            assert np.array_equal(y, g[p + "y"]), k
            assert np.array_equal(dx, g[p + "dx"]), k
            assert np.array_equal(dW, g[p + "dW"]), k
        else:           # the reference's N=2 instantiation is contracted differently by its compiler: 1-2 ulp
            assert _rel(y, g[p + "y"]) < 1e-6 and _rel(dx, g[p + "dx"]) < 1e-6 and _rel(dW, g[p + "dW"]) < 1e-6


def test_golden_differentiable_lut():
    g = np.load(os.path.join(GOLD, "differentiable_lut.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        n, I, O, F, bit, binary_mode, lut_binarize, batch_norm = [int(v) for v in g[p + "meta"]]
        x, idx, W, dy, rm, rv = g[p + "x"], g[p + "idx"], g[p + "W"], g[p + "dy"], g[p + "rm"], g[p + "rv"]
        if batch_norm:
            if bit:
                y, mean, rstd, rm2, rv2 = oracle.bit_differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize)
                yi = oracle.bit_differentiable_lut_forward_inference(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize)
                dx, dW = oracle.bit_differentiable_lut_backward(n, x, dy, idx, W, F, g[p + "mean"], g[p + "rstd"], None, lut_binarize=lut_binarize)
                assert np.array_equal(y, g[p + "y"]) and np.array_equal(yi, g[p + "y_inf"]), k
            else:
                y, mean, rstd, rm2, rv2 = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize, binary_mode=binary_mode)
                yi = oracle.differentiable_lut_forward_inference(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize, binary_mode=binary_mode)
                dx, dW = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, g[p + "mean"], g[p + "rstd"], None, lut_binarize=lut_binarize, binary_mode=binary_mode)
                assert np.abs(y - g[p + "y"]).max() < 2e-6 and np.abs(yi - g[p + "y_inf"]).max() < 2e-6, k
            assert _rel(mean, g[p + "mean"]) < 1e-6 and _rel(rstd, g[p + "rstd"]) < 1e-5, k
            assert _rel(rm2, g[p + "rm_out"]) < 1e-6 and _rel(rv2, g[p + "rv_out"]) < 1e-6, k
            assert _rel(dx, g[p + "dx"]) < 1e-5 and _rel(dW, g[p + "dW"]) < 1e-5, k
        else:
            if bit:
                y = oracle.bit_bit_stochastic_lut_forward(n, x, idx, W, F, lut_binarize)
                dx, dW = oracle.bit_stochastic_lut_backward(n, x, dy, idx, W, F, None, lut_binarize)
                assert np.array_equal(y, g[p + "y"]), k
            else:
                y = oracle.differentiable_lut_forward_nobn(n, x, idx, W, F, lut_binarize=lut_binarize, binary_mode=binary_mode)
                dx, dW = oracle.stochastic_lut_backward(n, x, dy, idx, W, F, None, binary_mode, lut_binarize, 0.25, False)
                assert np.abs(y - g[p + "y"]).max() < 2e-6, k
            assert _rel(dx, g[p + "dx"]) < 1e-5 and _rel(dW, g[p + "dW"]) < 1e-5, k


def test_golden_binary_lut6_and_reverse_table():
    g = np.load(os.path.join(GOLD, "binary_lut6.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        I, O, F = [int(v) for v in g[p + "meta"]]
        y = oracle.binary_lut6_forward(g[p + "xbits"], g[p + "idx"], g[p + "table"], F)
        assert np.array_equal(y, g[p + "y"])
        yw = oracle.binary_lut6_forward(g[p + "xbits"], g[p + "idx"], g[p + "table"], F, words=True)
        assert np.array_equal(synth.unpack_bits(yw, F), synth.unpack_bits(g[p + "y"], F))
        assert np.array_equal(oracle.reverse_table(6, g[p + "idx"], I), g[p + "rev"])


# ------------------------------------------------------------------ 2. the compiled reference, fresh inputs

needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref/libbbref.so not built here")


@needs_ref
@pytest.mark.parametrize("shape", [(6, 1, 1), (14, 16, 8), (14, 1024, 8), (14, 1024, 3), (13, 17, 1529)])   # tests/gtest/StochasticLutNTest.cpp:235-246
@pytest.mark.parametrize("lut_binarize", [0, 1])
def test_ref_stochastic_lut6(shape, lut_binarize):
    I, O, F = shape
    rng = np.random.default_rng(I * 1000 + O + F)
    for binary_mode in (0, 1):
        for simd in (1, 0):
            idx = synth.wiring(rng, I, O)
            W = synth.lut_tables(rng, O, 6, -0.2, 1.2)
            x = synth.uniform_frames(rng, I, F, stride=F, lo=-0.1, hi=1.1)
            dy = synth.normal_frames(rng, O, F, stride=F)
            dW0 = rng.standard_normal((O, 64)).astype(np.float32)
            r = oracle.ref_stochastic_lut(6, x, idx, W, dy=dy, dW_init=dW0, binary_mode=binary_mode, lut_binarize=lut_binarize, host_simd=simd)
            Wc = oracle.vector_clamp(W)
            use_simd = bool(simd) and F % 8 == 0          # include/bb/StochasticLutN.h:505-506
            y = oracle.stochastic_lut_forward(6, x, idx, Wc, F, binary_mode, lut_binarize, 0.25, use_simd)
            dx, dW = oracle.stochastic_lut_backward(6, x, dy, idx, Wc, F, dW0, binary_mode, lut_binarize, 0.25, use_simd)
            assert np.array_equal(Wc, r["W"]) and np.array_equal(y, r["y"])
            assert np.array_equal(dx, r["dx"]) and np.array_equal(dW, r["dW"])


@needs_ref
def test_ref_binary_lut6_and_reverse():
    rng = np.random.default_rng(7)
    for (I, O, F) in [(16, 16, 32), (100, 64, 2048), (33, 7, 257)]:
        idx = synth.wiring(rng, I, O)
        T = synth.truth_tables(rng, O)
        xb = synth.bernoulli_bits(rng, I, F)
        y = oracle.binary_lut6_forward(xb, idx, T, F)
        for simd in (0, 1):
            r = oracle.ref_binary_lut6(xb, idx, T, F, simd)
            assert np.array_equal(synth.unpack_bits(y, F), synth.unpack_bits(r, F))
        assert np.array_equal(oracle.reverse_table(6, idx, I), oracle.ref_reverse_table6(idx, I))


@needs_ref
@pytest.mark.parametrize("n", [6, 4])
def test_ref_differentiable_lut(n):
    rng = np.random.default_rng(11 + n)
    for (I, O, F) in [(20, 16, 39), (40, 32, 1024)]:
        for (bit, binary_mode) in [(0, 1), (0, 0), (1, 1)]:
            idx = synth.wiring(rng, I, O, n)
            W = synth.lut_tables(rng, O, n)
            dy = synth.normal_frames(rng, O, F, stride=F)
            rm = rng.random(O).astype(np.float32); rv = (rng.random(O) + 0.5).astype(np.float32)
            if bit:
                x = synth.bernoulli_bits(rng, I, F)
                r = oracle.ref_differentiable_lut(n, x, idx, W, rm, rv, dy=dy, bit_input=True, frame_size=F)
                y, mean, rstd, rm2, rv2 = oracle.bit_differentiable_lut_forward_training(n, x, idx, W, F, rm, rv)
                dx, dW = oracle.bit_differentiable_lut_backward(n, x, dy, idx, W, F, r["mean"], r["rstd"])
                assert np.array_equal(synth.unpack_bits(y, F), synth.unpack_bits(r["y"], F))
            else:
                x = synth.uniform_frames(rng, I, F, stride=F, lo=-0.1, hi=1.1)
                r = oracle.ref_differentiable_lut(n, x, idx, W, rm, rv, dy=dy, binary_mode=binary_mode)
                y, mean, rstd, rm2, rv2 = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, binary_mode=binary_mode)
                dx, dW = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, r["mean"], r["rstd"], binary_mode=binary_mode)
                assert np.abs(y - r["y"]).max() < 2e-6
            assert _rel(mean, r["mean"]) < 1e-6 and _rel(rstd, r["rstd"]) < 1e-5
            assert _rel(dx, r["dx"]) < 1e-5 and _rel(dW, r["dW"]) < 1e-5


# ------------------------------------------------------------------ 3. what the mathematics fixes

def _brute(n, x, idx, W, dy):
    """fp64 evaluation of include/bb/StochasticOperation.h:95-152 with numpy broadcasting."""
    O = idx.shape[0]; I, F = x.shape
    xs = np.clip(x.astype(np.float64), 0, 1)[idx]                       # [O, n, F]
    W = W.astype(np.float64); dy = dy.astype(np.float64)
    y = np.zeros((O, F)); dW = np.zeros((O, 1 << n)); dxs = np.zeros((O, n, F))
    for i in range(1 << n):
        fac = [xs[:, j] if (i >> j) & 1 else 1 - xs[:, j] for j in range(n)]
        p = np.prod(fac, axis=0)
        y += W[:, i:i + 1] * p
        dW[:, i] = (dy * p).sum(1)
        for k in range(n):
            pk = np.prod([fac[j] for j in range(n) if j != k], axis=0) if n > 1 else 1.0
            dxs[:, k] += (W[:, i:i + 1] if (i >> k) & 1 else -W[:, i:i + 1]) * pk * dy
    dx = np.zeros((I, F))
    for o in range(O):
        for k in range(n):
            dx[idx[o, k]] += dxs[o, k]
    return np.clip(y, 0, 1), dx, dW


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("simd", [0, 1])
def test_brute_force_fp64(n, simd):
    rng = np.random.default_rng(n)
    I, O, F = 12, 10, 48
    idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
    x = synth.uniform_frames(rng, I, F, stride=F); dy = synth.normal_frames(rng, O, F, stride=F)
    yb, dxb, dWb = _brute(n, x, idx, W, dy)
    y = oracle.stochastic_lut_forward(n, x, idx, W, F, simd=simd)
    dx, dW = oracle.stochastic_lut_backward(n, x, dy, idx, W, F, simd=simd)
    assert np.abs(y - yb).max() < 2e-6 and _rel(dx, dxb) < 1e-5 and _rel(dW, dWb) < 1e-5


@pytest.mark.parametrize("n", [2, 4, 6])
def test_corner_inputs_select_table_entries(n):
    # x in {0,1}^n  =>  y = W[sum_j x_j << j] exactly (input j is index bit j)
    rng = np.random.default_rng(3)
    NN = 1 << n
    x = np.array([[(f >> j) & 1 for f in range(NN)] for j in range(n)], np.float32)    # node j, frame f
    idx = np.arange(n, dtype=np.int32)[None, :]
    W = synth.lut_tables(rng, 1, n)
    for simd in (0, 1):
        y = oracle.stochastic_lut_forward(n, x, idx, W, NN, simd=simd)
        assert np.array_equal(y[0], W[0])
    # lut_binarize: W -> (W > 0.5)
    y = oracle.stochastic_lut_forward(n, x, idx, W, NN, lut_binarize=True)
    assert np.array_equal(y[0], (W[0] > 0.5).astype(np.float32))
    # binary mode: x -> 0.5 +- 0.25; every table equal to c gives c
    Wc = np.full((1, NN), 0.375, np.float32)
    y = oracle.stochastic_lut_forward(n, x, idx, Wc, NN, input_binary=True)
    assert np.abs(y - 0.375).max() < 1e-6


def test_sum_rules_and_finite_differences():
    rng = np.random.default_rng(5)
    n, I, O, F = 6, 16, 12, 64
    idx = synth.wiring(rng, I, O); W = synth.lut_tables(rng, O)
    x = synth.uniform_frames(rng, I, F, stride=F, lo=0.05, hi=0.95); dy = synth.normal_frames(rng, O, F, stride=F)
    dx, dW = oracle.stochastic_lut_backward(n, x, dy, idx, W, F)
    # sum_i prod_i = 1  =>  sum_i dW[o, i] = sum_f dy[o, f]
    assert np.abs(dW.sum(1) - dy.astype(np.float64).sum(1)).max() < 1e-4
    # multilinearity: dy/dx_k = y(x_k = 1) - y(x_k = 0); dx[in] is the sum over its fan-out
    ref = np.zeros((I, F))
    for o in range(O):
        for k in range(n):
            x1 = x.copy(); x0 = x.copy()
            x1[idx[o, k]] = 1.0; x0[idx[o, k]] = 0.0
            y1 = oracle.stochastic_lut_forward(n, x1, idx[o:o + 1], W[o:o + 1], F)[0].astype(np.float64)
            y0 = oracle.stochastic_lut_forward(n, x0, idx[o:o + 1], W[o:o + 1], F)[0].astype(np.float64)
            ref[idx[o, k]] += dy[o] * (y1 - y0)
    assert np.abs(dx - ref).max() < 1e-5
    # dW accumulates on top of what is there
    dx2, dW2 = oracle.stochastic_lut_backward(n, x, dy, idx, W, F, dW_init=dW)
    assert _rel(dW2, 2 * dW.astype(np.float64)) < 1e-6


def test_binary_lut6_equals_stochastic_lut_on_bits():
    rng = np.random.default_rng(9)
    I, O, F = 40, 24, 200
    idx = synth.wiring(rng, I, O); T = synth.truth_tables(rng, O)
    xb = synth.bernoulli_bits(rng, I, F)
    y = synth.unpack_bits(oracle.binary_lut6_forward(xb, idx, T, F), F)
    W = np.array([[(int(np.uint32(T[o, b >> 5])) >> (b & 31)) & 1 for b in range(64)] for o in range(O)], np.float32)
    ys = oracle.stochastic_lut_forward(6, synth.unpack_bits(xb, F).astype(np.float32), idx, W, F, simd=False)
    assert np.array_equal(y, ys.astype(np.uint8))
    # known answer in the style of tests/gtest/BinaryLutTest.cpp:12-116: node wired to inputs 0..5, table bit k set only at k=37
    T1 = np.zeros((1, 2), np.int32); T1[0, 1] = 1 << (37 - 32)
    x1 = synth.pack_bits(np.array([[(f >> j) & 1 for f in range(64)] for j in range(6)], np.uint8))
    y1 = synth.unpack_bits(oracle.binary_lut6_forward(x1, np.arange(6, dtype=np.int32)[None], T1, 64), 64)[0]
    assert y1.sum() == 1 and y1[37] == 1


def test_batchnorm_statistics_and_gradient_invariants():
    rng = np.random.default_rng(13)
    n, I, O, F = 6, 24, 10, 256
    idx = synth.wiring(rng, I, O); W = synth.lut_tables(rng, O)
    x = synth.uniform_frames(rng, I, F, stride=F); dy = synth.normal_frames(rng, O, F, stride=F)
    rm = np.zeros(O, np.float32); rv = np.ones(O, np.float32)
    gamma, beta, mom = 0.3, 0.5, 0.9
    y, mean, rstd, rm2, rv2 = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, gamma, beta, mom, binary_mode=False)
    # raw LUT output (not clamped): huge window on a no-BN, non-binary evaluation is not available -> fp64 restatement
    xs = np.clip(x.astype(np.float64), 0, 1)[idx]
    raw = np.zeros((O, F))
    for i in range(64):
        raw += W[:, i:i + 1].astype(np.float64) * np.prod([xs[:, j] if (i >> j) & 1 else 1 - xs[:, j] for j in range(6)], axis=0)
    m = raw.mean(1); v = np.maximum(1e-5, (raw ** 2).mean(1) - m ** 2)
    assert np.abs(mean - m).max() < 1e-6 and _rel(rstd, 1 / np.sqrt(v)) < 1e-5
    assert _rel(rm2, m * (1 - mom)) < 1e-5 and _rel(rv2, mom + v * (1 - mom)) < 1e-6
    t = (raw - m[:, None]) / np.sqrt(v)[:, None] * gamma + beta
    assert np.abs(y - np.clip(t, 0, 1)).max() < 1e-5
    # gradient through batch-norm is orthogonal to constants and to the centred signal when no frame is gated:
    # make the hard-tanh window inactive with small gamma
    g2 = 0.01
    y2, mean2, rstd2, _, _ = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, g2, beta, mom, binary_mode=False)
    dx, dW = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, mean2, rstd2, gamma=g2, beta=beta, binary_mode=False)
    # dW[o] = sum_f dyhat * prod_i, and sum_i prod_i = 1, so sum_i dW[o,i] = sum_f dyhat = 0 (BN removes the mean)
    assert np.abs(dW.sum(1)).max() < 1e-4
    # sum_i W_i prod_i = raw, so sum_i W[o,i] dW[o,i] = sum_f dyhat*raw = sum_f dyhat*(raw-mean) = 0 (BN removes the scale)
    assert np.abs((W.astype(np.float64) * dW).sum(1)).max() < 1e-4
