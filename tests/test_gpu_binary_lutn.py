"""GPU parity of BinaryLutN<N> packed inference for N = 2 .. 6 (bbhip_bit_BinaryLutN_Forward): bit-exact against the CPU oracle and
against vectors written by the reference's own class; equal to StochasticLut<N> with a 0 / 1 table on the same bits."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "binary_lutn.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def tables(rng, O, n):
    if n == 6:
        return synth.truth_tables(rng, O)
    return rng.integers(0, 1 << (1 << n), (O, 1), dtype=np.int64).astype(np.uint32).view(np.int32)


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("shape", [(16, 16, 32), (70, 33, 1000), (8, 5, 7), (6, 1, 1), (300, 1000, 64 * 32 * 3 + 5), (64, 130, 131072 + 37)])
def test_bit_exact(ops, n, shape):
    I, O, F = shape
    rng = np.random.default_rng(I + O + F + n)
    stride = synth.frame_stride_bit(F)
    idx = synth.wiring(rng, I, O, n); T = tables(rng, O, n)
    xb = synth.bernoulli_bits(rng, I, F, stride)
    y = ops.binary_lutn_forward(n, dev(xb), dev(idx), dev(T), F)
    assert np.array_equal(host(y), oracle.binary_lutn_forward(n, xb, idx, T, F))        # padding bits and words are zero on both sides


def test_reference_vectors_on_gpu(ops):
    for k in range(int(GOLD["count"][0])):
        p = "c%d_" % k
        n, I, O, F = [int(v) for v in GOLD[p + "meta"]]
        y = ops.binary_lutn_forward(n, dev(GOLD[p + "xbits"]), dev(GOLD[p + "idx"]), dev(GOLD[p + "table"]), F)
        assert np.array_equal(host(y), GOLD[p + "y"]), (k, n)


@pytest.mark.parametrize("n", [2, 3, 4, 5])
def test_equals_the_stochastic_lut_on_bits(ops, n):
    """the same layer as a StochasticLut<n> with W in {0, 1} and bit inputs mapped to 0 / 1 (bias 0.5): y > 0.5 reproduces the table"""
    rng = np.random.default_rng(60 + n)
    I, O, F = 40, 24, 4096 + 70
    idx = synth.wiring(rng, I, O, n); T = tables(rng, O, n)
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
    W = np.array([[(int(np.uint32(T[o, 0])) >> b) & 1 for b in range(1 << n)] for o in range(O)], np.float32)
    y = ops.binary_lutn_forward(n, dev(xb), dev(idx), dev(T), F)
    yb = ops.bit_bit_stochastic_lut_forward(n, dev(xb), dev(idx), dev(W), F, bias=0.5)
    assert np.array_equal(synth.unpack_bits(host(yb), F), synth.unpack_bits(host(y), F))


def test_rejected_arguments(ops):
    import torch
    x = torch.zeros((8, 8), dtype=torch.int32, device="cuda")
    idx = torch.zeros((4, 7), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError):
        from binarybrain_amd.capi import lib, check
        from binarybrain_amd.ops import ptr
        check(lib().bbhip_bit_BinaryLutN_Forward(7, ptr(x), ptr(x), ptr(idx), ptr(idx), 4, 64, 8, None))
