"""The oracle's StochasticBatchNormalization, pinned without a GPU: vectors written by the reference's own host class
(tests/golden/bn.npz), the compiled reference where oracle/_ref is present, textbook statistics in float64 and the two sums that
the gradient of a normalisation must make vanish.

The reference build contracts multiply-add pairs where the compiler chooses to; the oracle keeps every operation apart.  The two
therefore agree to a few units in the last place of the largest term, not bit for bit: 1e-6 relative for y and the statistics,
and for dx 1e-6 of gamma * |dy| * rstd, the size of the terms that cancel in it (a row without variance has rstd = 1e7)."""
import os

import numpy as np
import pytest

import oracle

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "bn.npz"))
F32 = np.float32


def close(a, b, scale=1.0, tol=1e-6):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return np.all(np.abs(a - b) <= tol * (np.maximum(np.abs(b), scale)))


def dx_scale(dy, rstd, gamma):
    return (abs(gamma) * np.abs(dy).max(axis=1) * rstd)[:, None] + 1.0


def check_against(r, x, dy, rm, rv, gamma, beta, momentum):
    nodes, F = x.shape
    y, mean, rstd, rm2, rv2 = oracle.stochastic_bn_forward_training(x, rm, rv, gamma, beta, momentum, F)
    assert np.array_equal(mean, r["mean"])                          # a plain sum in frame order: no room for contraction
    assert close(rstd, r["rstd"]) and close(rm2, r["running_mean"]) and close(rv2, r["running_var"])
    assert np.all(np.abs(y - r["y"]) <= 1e-6 * (np.abs((x - mean[:, None]) * rstd[:, None] * gamma) + 1.0))
    # the backward pass from the reference's own statistics, so that only its own arithmetic is compared
    dx = oracle.stochastic_bn_backward(x, dy, r["mean"], r["rstd"], gamma, F)
    assert np.all(np.abs(dx.astype(np.float64) - r["dx"]) <= 1e-6 * dx_scale(dy, r["rstd"], gamma) * max(1.0, np.abs(x).max()))
    assert np.array_equal(oracle.stochastic_bn_reforward(x, mean, rstd, gamma, beta, F), y)


def test_reference_vectors():
    for k in range(int(GOLD["count"][0])):
        p = "b%d_" % k
        momentum, gamma, beta = [float(v) for v in GOLD[p + "scalars"]]
        r = {key: GOLD[p + key] for key in ("y", "mean", "rstd", "running_mean", "running_var", "dx")}
        check_against(r, GOLD[p + "x"], GOLD[p + "dy"], GOLD[p + "running_mean_in"], GOLD[p + "running_var_in"], gamma, beta, momentum)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_against_compiled_reference():
    rng = np.random.default_rng(11)
    for (nodes, F, momentum, gamma, beta) in [(12, 100, 0.9, 0.2, 0.5), (4, 513, 0.7, 0.3, 0.45), (30, 32, 0.999, 1.5, -0.25)]:
        x = rng.random((nodes, F)).astype(F32)
        dy = rng.standard_normal((nodes, F)).astype(F32)
        rm = rng.standard_normal(nodes).astype(F32); rv = (rng.random(nodes) + 0.1).astype(F32)
        r = oracle.ref_stochastic_bn(x, rm, rv, gamma, beta, momentum, train=True, dy=dy)
        check_against(r, x, dy, rm, rv, gamma, beta, momentum)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_inference_against_compiled_reference():
    # The reference's generic inference pass takes its offset from the mean of the last training batch.  After one training pass
    # with momentum 0 the running mean IS that batch mean, so there both readings coincide and the formula can be compared.
    rng = np.random.default_rng(12)
    nodes, F, gamma, beta = 9, 77, 0.2, 0.5
    x = rng.random((nodes, F)).astype(F32)
    first = oracle.ref_stochastic_bn(x, np.zeros(nodes, F32), np.ones(nodes, F32), gamma, beta, 0.0, train=True)
    assert np.array_equal(first["running_mean"], first["mean"])
    y = oracle.stochastic_bn_forward_inference(x, first["running_mean"], first["running_var"], gamma, beta, F)
    # with these statistics inference repeats the training output
    assert close(y, first["y"], tol=2e-6)
    # and with foreign statistics it is the textbook affine map
    rm = rng.standard_normal(nodes).astype(F32); rv = (rng.random(nodes) + 0.1).astype(F32)
    y = oracle.stochastic_bn_forward_inference(x, rm, rv, gamma, beta, F)
    want = (x.astype(np.float64) - rm[:, None]) / (np.sqrt(rv.astype(np.float64))[:, None] + 1e-7) * gamma + beta
    assert np.abs(y - want).max() < 1e-5


def test_textbook_statistics():
    rng = np.random.default_rng(13)
    nodes, F, gamma, beta, momentum = 10, 400, 0.2, 0.5, 0.9
    x = (rng.standard_normal((nodes, F)) * 3 + 1).astype(F32)
    rm = rng.standard_normal(nodes).astype(F32); rv = (rng.random(nodes) + 0.5).astype(F32)
    y, mean, rstd, rm2, rv2 = oracle.stochastic_bn_forward_training(x, rm, rv, gamma, beta, momentum, F)
    x64 = x.astype(np.float64)
    assert np.abs(mean - x64.mean(axis=1)).max() < 1e-5
    var = x64.var(axis=1)                                           # the biased variance: divided by F, not F - 1
    assert np.abs(rstd - 1.0 / (np.sqrt(var) + 1e-7)).max() < 1e-5
    assert np.abs(rm2 - (rm * momentum + x64.mean(axis=1) * (1 - momentum))).max() < 1e-5
    assert np.abs(rv2 - (rv * momentum + var * (1 - momentum))).max() < 1e-5
    # the output has mean beta and deviation gamma in every row
    assert np.abs(y.astype(np.float64).mean(axis=1) - beta).max() < 1e-5
    assert np.abs(y.astype(np.float64).std(axis=1) - gamma).max() < 1e-5
    # a stride wider than the frame count: the padding is neither read nor written
    xs = np.full((nodes, F + 24), 7.0, F32); xs[:, :F] = x
    ys = oracle.stochastic_bn_forward_training(xs, rm, rv, gamma, beta, momentum, F)[0]
    assert np.array_equal(ys[:, :F], y) and np.all(ys[:, F:] == 0)


def test_gradient_against_float64_and_its_invariants():
    rng = np.random.default_rng(14)
    nodes, F, gamma = 6, 300, 0.35
    x = rng.random((nodes, F)).astype(F32)
    dy = rng.standard_normal((nodes, F)).astype(F32)
    _, mean, rstd, _, _ = oracle.stochastic_bn_forward_training(x, np.zeros(nodes, F32), np.ones(nodes, F32), gamma, 0.5, 0.9, F)
    dx = oracle.stochastic_bn_backward(x, dy, mean, rstd, gamma, F).astype(np.float64)
    # the gradient of y = gamma (x - mean(x)) / std(x) + beta, written out in float64 (eps left out: std >> 1e-7 here)
    x64 = x.astype(np.float64); g = dy.astype(np.float64) * gamma
    mu = x64.mean(axis=1, keepdims=True); sd = x64.std(axis=1, keepdims=True)
    xh = (x64 - mu) / sd
    want = (g - g.mean(axis=1, keepdims=True) - xh * (g * xh).mean(axis=1, keepdims=True)) / sd
    assert np.abs(dx - want).max() < 2e-5 * np.abs(want).max()
    # shifting or scaling a row does not change the output, so the gradient is orthogonal to both directions
    assert np.abs(dx.sum(axis=1)).max() < 1e-4 * np.abs(dx).sum(axis=1).max()
    assert np.abs((dx * (x64 - mu)).sum(axis=1)).max() < 1e-4 * np.abs(dx * (x64 - mu)).sum(axis=1).max()
    # and a finite difference of the float64 forward agrees
    def fwd(v):
        return ((v - v.mean(axis=1, keepdims=True)) / v.std(axis=1, keepdims=True) * gamma * dy).sum()
    for (n, f) in [(0, 0), (3, 17), (5, 299)]:
        e = np.zeros_like(x64); e[n, f] = 1e-6
        assert abs((fwd(x64 + e) - fwd(x64 - e)) / 2e-6 - dx[n, f]) < 1e-4 * max(1.0, abs(dx[n, f]))
