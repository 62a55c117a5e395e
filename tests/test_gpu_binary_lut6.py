"""GPU parity of BinaryLut6 packed inference: bit-exact against the CPU oracle and the reference's own vectors."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


# (the last two shapes are large enough for the library to put four, resp. two, nodes on a wavefront; their node counts leave
# a last wavefront with nodes to skip, and the last words of their rows are partial)
@pytest.mark.parametrize("shape", [(16, 16, 32), (64, 32, 512), (70, 33, 1000), (8, 5, 7), (6, 1, 1), (300, 1000, 64 * 32 * 3 + 5),
                                   (64, 1030, 131072 + 37), (64, 517, 131072 + 2049)])
def test_bit_exact(ops, shape):
    I, O, F = shape
    rng = np.random.default_rng(I + O + F)
    stride = synth.frame_stride_bit(F)
    idx = synth.wiring(rng, I, O); T = synth.truth_tables(rng, O)
    xb = synth.bernoulli_bits(rng, I, F, stride)
    y = ops.binary_lut6_forward(dev(xb), dev(idx), dev(T), F)
    assert np.array_equal(host(y), oracle.binary_lut6_forward(xb, idx, T, F))      # padding bits and words are zero on both sides


def test_golden_vectors_on_gpu(ops):
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "binary_lut6.npz"))
    for k in range(int(g["count"][0])):
        p = "c%d_" % k
        I, O, F = [int(v) for v in g[p + "meta"]]
        y = ops.binary_lut6_forward(dev(g[p + "xbits"]), dev(g[p + "idx"]), dev(g[p + "table"]), F)
        assert np.array_equal(host(y), g[p + "y"])


def test_known_answer(ops):
    # node wired to inputs 0..5, frame f carries the 6-bit pattern f: y(f) = table bit f  (tests/gtest/BinaryLutTest.cpp:12-116 semantics)
    import torch
    x = synth.pack_bits(np.array([[(f >> j) & 1 for f in range(64)] for j in range(6)], np.uint8))
    T = np.array([[0x12345678, np.int32(np.uint32(0x9abcdef0))]], dtype=np.int64).astype(np.uint32).view(np.int32).reshape(1, 2)
    y = host(ops.binary_lut6_forward(dev(x), dev(np.arange(6, dtype=np.int32)[None]), dev(T), 64))
    assert np.array_equal(y.view(np.uint32)[0], T.view(np.uint32)[0])


def test_full_size_against_oracle_slice_and_stochastic_lut(ops):
    """8192 -> 16384 nodes, 262144 frames: a slice of nodes against the oracle; equality with StochasticLut on {0,1} data."""
    import torch
    rng = np.random.default_rng(4)
    I, O, F = 8192, 16384, 262144
    idx = synth.wiring(rng, I, O); T = synth.truth_tables(rng, O)
    xb = synth.bernoulli_bits(rng, I, F)
    y = ops.binary_lut6_forward(dev(xb), dev(idx), dev(T), F)
    sel = np.arange(0, O, 509)                  # every position of a node within the group that shares a wavefront
    y_ref = oracle.binary_lut6_forward(xb, idx[sel], T[sel], F, words=True)
    yh = host(y)
    assert np.array_equal(yh[sel], y_ref)
    # every node: over the first and over the last 8192 frames (256 words each; a node's words do not depend on one another)
    for w0 in (0, F // 32 - 256):
        part = np.ascontiguousarray(xb[:, w0:w0 + 256])
        assert np.array_equal(yh[:, w0:w0 + 256], oracle.binary_lut6_forward(part, idx, T, 8192, words=True)), w0
    # the same layer as a StochasticLut with W in {0,1} and bit inputs mapped to 0/1 (bias 0.5): y > 0.5 reproduces the table
    sel2 = sel[:8]
    W = np.array([[(int(np.uint32(T[o, b >> 5])) >> (b & 31)) & 1 for b in range(64)] for o in sel2], np.float32)
    yb = ops.bit_bit_stochastic_lut_forward(6, dev(xb), dev(idx[sel2]), dev(W), F, bias=0.5)
    assert np.array_equal(host(yb), yh[sel2])
