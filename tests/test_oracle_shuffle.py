"""The oracle's Shuffle, pinned without a GPU: vectors written by the reference's own host class (tests/golden/pooling.npz, keys
s*), the compiled reference where oracle/_ref is present, the known answer of the reference's test (tests/gtest/ShuffleTest.cpp:9-60)
and numpy's transpose.  A permutation of rows: bit-exact."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "pooling.npz"))
F32 = np.float32


def valid(words, frames):
    return synth.unpack_bits(words, frames)


def test_reference_vectors():
    for k in range(int(GOLD["shuffle_count"][0])):
        q = "s%d_" % k
        nodes, unit, F = [int(v) for v in GOLD[q + "geom"]]
        assert np.array_equal(oracle.shuffle_forward(GOLD[q + "x"], unit), GOLD[q + "y"]), k
        assert np.array_equal(oracle.shuffle_backward(GOLD[q + "dy"], unit), GOLD[q + "dx"]), k
        assert np.array_equal(oracle.shuffle_forward(GOLD[q + "xbits"], unit), GOLD[q + "y_bits"]), k
        assert np.array_equal(oracle.shuffle_backward(GOLD[q + "dybits"], unit), GOLD[q + "dx_bits"]), k


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
def test_against_compiled_reference():
    rng = np.random.default_rng(71)
    for nodes, unit, F in ((12, 4, 5), (30, 5, 33), (64, 1, 7), (64, 64, 7), (35, 7, 70), (1024, 32, 100), (6, 2, 1)):
        x = rng.standard_normal((nodes, F)).astype(F32)
        dy = rng.standard_normal((nodes, F)).astype(F32)
        y, dx, _ = oracle.ref_shuffle(x, unit, F, dy=dy)
        assert np.array_equal(oracle.shuffle_forward(x, unit), y) and np.array_equal(oracle.shuffle_backward(dy, unit), dx), (nodes, unit, F)
        xb = synth.bernoulli_bits(rng, nodes, F); dyb = synth.bernoulli_bits(rng, nodes, F)
        yb, dxb, _ = oracle.ref_shuffle(xb, unit, F, bit=True, dy=dyb)         # bits past the last frame: whatever the buffers held
        assert np.array_equal(valid(oracle.shuffle_forward(xb, unit), F), valid(yb, F)), (nodes, unit, F)
        assert np.array_equal(valid(oracle.shuffle_backward(dyb, unit), F), valid(dxb, F)), (nodes, unit, F)


def test_known_answer_of_the_reference_test():
    # tests/gtest/ShuffleTest.cpp:9-60: 6 nodes in units of 3, frames 0 and 1 hold 11..16 and 21..26
    x = np.array([[11, 21], [12, 22], [13, 23], [14, 24], [15, 25], [16, 26]], F32)
    y = oracle.shuffle_forward(x, 3)
    assert y[:, 0].tolist() == [11, 13, 15, 12, 14, 16] and y[:, 1].tolist() == [21, 23, 25, 22, 24, 26]
    assert np.array_equal(oracle.shuffle_backward(y, 3), x)


def test_numpy_restatements():
    rng = np.random.default_rng(72)
    for nodes, unit, stride in ((84, 7, 70), (60, 12, 3), (16, 16, 9), (16, 1, 9), (210, 14, 33)):
        x = rng.integers(-2**31, 2**31, (nodes, stride)).astype(np.int32)
        group = nodes // unit
        y = oracle.shuffle_forward(x, unit)
        assert np.array_equal(y, x.reshape(unit, group, stride).transpose(1, 0, 2).reshape(nodes, stride))   # rows [unit][group] -> [group][unit]
        assert np.array_equal(oracle.shuffle_backward(y, unit), x)                                           # backward undoes forward
        assert np.array_equal(oracle.shuffle_forward(oracle.shuffle_backward(x, unit), unit), x)
        assert np.array_equal(oracle.shuffle_backward(x, unit), oracle.shuffle_forward(x, group))            # the inverse deals by the other extent
        # a permutation: <forward(a), b> = <a, backward(b)>, the property a gradient must have
        a = rng.standard_normal((nodes, stride)).astype(F32); b = rng.standard_normal((nodes, stride)).astype(F32)
        assert np.array_equal(np.sort(oracle.shuffle_forward(a, unit), axis=None), np.sort(a, axis=None))
        lhs = (oracle.shuffle_forward(a, unit).astype(np.float64) * b).sum(); rhs = (a.astype(np.float64) * oracle.shuffle_backward(b, unit)).sum()
        assert abs(lhs - rhs) <= 1e-9 * max(1.0, abs(lhs))
