"""The oracle's elementwise vector operations and Adam step, pinned without a GPU:
vectors written by the reference's own host code (tests/golden/adam.npz), the compiled reference itself where
oracle/_ref is present, fp32 closed forms evaluated with numpy, the update model of the reference's optimizer test
(tests/gtest/OptimizerAdamTest.cpp:10-40) and the textbook form of Adam in fp64."""
import os

import numpy as np
import pytest

import oracle

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "adam.npz"))
F32 = np.float32


def _ulp_close(a, b, ulps):
    a = np.asarray(a, F32); b = np.asarray(b, F32)
    tol = ulps * np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(F32))
    return bool(np.all(np.abs(a.astype(np.float64) - b.astype(np.float64)) <= tol))


def _close_at(a, b, scale, ulps=2):
    """|a - b| within `ulps` units in the last place of `scale` (the largest intermediate of the expression: where two
    terms cancel, a fused multiply-add in the reference build shifts the result by an ulp of the terms, not of the sum)."""
    tol = ulps * np.spacing(np.asarray(scale, F32))
    return bool(np.all(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)) <= tol))


def test_vector_ops_against_reference_vectors():
    x, y, pos = GOLD["vx"], GOLD["vy"], GOLD["vpos"]
    a, b, c, d = [float(v) for v in GOLD["coef"]]
    # single-rounding operations and selections: bit-exact
    assert np.array_equal(oracle.vector_op("sqrt", pos), GOLD["sqrt"])
    assert np.array_equal(oracle.vector_op("min", x, y), GOLD["min"])
    assert np.array_equal(oracle.vector_op("min_v", x, None, 0.3), GOLD["min_v"])
    assert np.array_equal(oracle.vector_op("max", x, y), GOLD["max"])
    assert np.array_equal(oracle.vector_op("max_v", x, None, 0.3), GOLD["max_v"])
    # multi-operation expressions: the reference build may contract a*x+b*y into a fused multiply-add
    assert _close_at(oracle.vector_op("add_ex", x, y, a, b, c), GOLD["add_ex"], np.abs(a * x) + np.abs(b * y) + abs(c))
    assert _close_at(oracle.vector_op("mul_ex", x, y, a, b), GOLD["mul_ex"], np.abs(a * x * y) + abs(b))
    assert _close_at(oracle.vector_op("div_ex", x, pos, a, b, c, d), GOLD["div_ex"], (np.abs(a * x) + abs(b)) / (c * pos + d))
    assert _ulp_close(oracle.vector_op("exp", x), GOLD["exp"], 2)


def test_vector_ops_closed_forms():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(1000) * 4).astype(F32); y = (rng.standard_normal(1000) * 4).astype(F32)
    a, b, c, d = F32(0.7), F32(-1.3), F32(0.11), F32(5.0)
    # numpy evaluates each fp32 operation with one rounding: the same sequence, written independently
    assert np.array_equal(oracle.vector_op("add_ex", x, y, a, b, c), (a * x + b * y) + c)
    assert np.array_equal(oracle.vector_op("mul_ex", x, y, a, b), (a * x) * y + b)
    assert np.array_equal(oracle.vector_op("div_ex", x, y, a, b, c, d), (a * x + b) / (c * y + d))
    assert np.array_equal(oracle.vector_op("sqrt", np.abs(x)), np.sqrt(np.abs(x)))
    assert np.allclose(oracle.vector_op("exp", x), np.exp(x.astype(np.float64)), rtol=3e-7, atol=0)
    assert np.array_equal(oracle.vector_op("min", x, y), np.minimum(x, y))
    assert np.array_equal(oracle.vector_op("max_v", x, None, 0.25), np.maximum(x, F32(0.25)))
    # identities the Tensor operators are built from (include/bb/Tensor.h:745-797)
    assert np.array_equal(oracle.vector_op("add_ex", x, y, 1, -1, 0), x - y)
    assert np.array_equal(oracle.vector_op("div_ex", x, y, 1, 0, 0, 2.0), x / F32(2.0))
    # std::min / std::max: a NaN in the second operand is dropped, in the first it propagates
    n = np.array([np.nan, 1.0], F32); o = np.array([1.0, np.nan], F32)
    r = oracle.vector_op("min", n, o)
    assert np.isnan(r[0]) and r[1] == 1.0


def test_adam_against_reference_vectors():
    for k in range(int(GOLD["adam_count"][0])):
        lr, b1, b2 = GOLD["a%d_hyper" % k]
        p, m, v = oracle.adam_steps(GOLD["a%d_p0" % k], list(GOLD["a%d_g" % k]), lr, b1, b2)
        # the reference composes the update from its tensor operators with unit coefficients, so every operation is
        # rounded once (nothing for its compiler to fuse): bit-exact
        assert np.array_equal(p, GOLD["a%d_p" % k]), k
        if p.size > 8:
            assert p[3] == GOLD["a%d_p0" % k][3]            # zero gradient: m = v = 0, the parameter does not move


def test_adam_matches_the_reference_test_model_and_fp64():
    """ModelAdam of the reference's optimizer test: scalar m, v, lr_t recomputed from beta^t each step."""
    rng = np.random.default_rng(11)
    lr, beta1, beta2 = 0.001, 0.9, 0.999
    g = (rng.standard_normal((25, 50)) * 2.0 + 0.0001).astype(F32)
    p0 = rng.standard_normal(50).astype(F32)
    p, m, v = oracle.adam_steps(p0, list(g), lr, beta1, beta2)
    # the test's model, in fp32 with the same association
    pm = p0.copy(); mm = np.zeros(50, F32); vm = np.zeros(50, F32); b1 = F32(beta1); b2 = F32(beta2)
    for t in range(25):
        lr_t = F32(F32(lr) * np.sqrt(F32(1) - b2, dtype=F32)) / (F32(1) - b1)
        mm = mm + (F32(1) - F32(beta1)) * (g[t] - mm)
        vm = vm + (F32(1) - F32(beta2)) * (g[t] * g[t] - vm)
        pm = pm - lr_t * mm / (np.sqrt(vm) + F32(1e-7))
        b1 = F32(b1 * F32(beta1)); b2 = F32(b2 * F32(beta2))
    assert np.array_equal(p, pm) and np.array_equal(m, mm) and np.array_equal(v, vm)
    # textbook Adam (Kingma & Ba, algorithm 1 with the folded bias correction) in fp64
    p64 = p0.astype(np.float64); m64 = np.zeros(50); v64 = np.zeros(50)
    for t in range(1, 26):
        m64 = beta1 * m64 + (1 - beta1) * g[t - 1]; v64 = beta2 * v64 + (1 - beta2) * g[t - 1].astype(np.float64) ** 2
        p64 -= lr * np.sqrt(1 - beta2 ** t) / (1 - beta1 ** t) * m64 / (np.sqrt(v64) + 1e-7)
    assert np.allclose(p, p64, rtol=0, atol=2e-6)
    # first step moves every parameter by lr against the sign of its gradient
    p1, _, _ = oracle.adam_steps(p0, [g[0]], lr, beta1, beta2)
    assert np.allclose(p1 - p0, -lr * np.sign(g[0]), rtol=1e-4, atol=0)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (reference tree absent)")
def test_against_compiled_reference():
    rng = np.random.default_rng(21)
    for size, steps in [(3, 4), (1000, 7)]:
        p0 = rng.standard_normal(size).astype(F32)
        g = (rng.standard_normal((steps, size)) * 1.5).astype(F32)
        p, _, _ = oracle.adam_steps(p0, list(g), 0.002, 0.85, 0.995)
        assert np.array_equal(p, oracle.ref_adam_steps(p0, list(g), 0.002, 0.85, 0.995))
    x = (rng.standard_normal(500) * 2).astype(F32); y = (rng.standard_normal(500) * 2).astype(F32)
    ya = np.abs(y) + 1
    for name, args, scale in [("add_ex", (x, y, 0.3, 1.7, -2.0), np.abs(0.3 * x) + np.abs(1.7 * y) + 2.0),
                              ("mul_ex", (x, y, 0.3, 1.7), np.abs(0.3 * x * y) + 1.7),
                              ("div_ex", (x, ya, 0.3, 1.7, 2.0, 0.5), (np.abs(0.3 * x) + 1.7) / (2.0 * ya + 0.5))]:
        assert _close_at(oracle.vector_op(name, *args), oracle.ref_vector_op(name, *args), scale), name
    for name, args in [("sqrt", (np.abs(x),)), ("exp", (x,)), ("min", (x, y)), ("max", (x, y)), ("min_v", (x, None, -0.2)), ("max_v", (x, None, -0.2))]:
        assert _ulp_close(oracle.vector_op(name, *args), oracle.ref_vector_op(name, *args), 2), name
