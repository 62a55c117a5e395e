"""The oracle's BinaryLutN<N> for N = 2 .. 6 (oracle_bit_BinaryLutN_Forward, a restatement of the generic loop of
include/bb/BinaryLutN.h:436-463) is pinned by: vectors written by the reference's own class (tests/golden/binary_lutn.npz), the reference
itself on fresh inputs where oracle/_ref is built, a numpy evaluation of the definition (y = table bit number sum_k x_k << k), and the
N = 6 restatement that the other tests pin."""
import os

import numpy as np
import pytest

import oracle
from binarybrain_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "binary_lutn.npz"))


def tables(rng, O, n):
    if n == 6:
        return synth.truth_tables(rng, O)
    return rng.integers(0, 1 << (1 << n), (O, 1), dtype=np.int64).astype(np.uint32).view(np.int32)


def by_definition(n, xb, idx, table, F):
    x = synth.unpack_bits(xb, F).astype(np.int64)                      # [I, F]
    index = sum(x[idx[:, k]] << k for k in range(n))                   # [O, F]
    t = table.view(np.uint32).astype(np.uint64)
    word = np.take_along_axis(t, (index >> 5).astype(np.int64), axis=1) if t.shape[1] > 1 else np.broadcast_to(t, index.shape)
    return ((word >> (index & 31).astype(np.uint64)) & 1).astype(np.uint8)


def test_reference_vectors():
    for k in range(int(GOLD["count"][0])):
        p = "c%d_" % k
        n, I, O, F = [int(v) for v in GOLD[p + "meta"]]
        y = oracle.binary_lutn_forward(n, GOLD[p + "xbits"], GOLD[p + "idx"], GOLD[p + "table"], F)
        assert np.array_equal(y, GOLD[p + "y"]), (k, n)


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6])
def test_definition_and_known_answers(n):
    rng = np.random.default_rng(100 + n)
    for (I, O, F) in [(12, 7, 70), (n, 1, 1 << n), (50, 40, 1000)]:
        idx = synth.wiring(rng, I, O, n); T = tables(rng, O, n)
        xb = synth.bernoulli_bits(rng, I, F, (F + 31) // 32)
        y = oracle.binary_lutn_forward(n, xb, idx, T, F)
        assert np.array_equal(synth.unpack_bits(y, F), by_definition(n, xb, idx, T, F))
        assert np.array_equal(y, synth.pack_bits(synth.unpack_bits(y, F), y.shape[1]))       # nothing behind the last frame
    # one node wired to inputs 0 .. n-1, frame f carries the n-bit pattern f: the output spells the table (tests/gtest/BinaryLutTest.cpp:12-116)
    F = 1 << n
    x = synth.pack_bits(np.array([[(f >> j) & 1 for f in range(F)] for j in range(n)], np.uint8))
    T = tables(rng, 1, n)
    y = oracle.binary_lutn_forward(n, x, np.arange(n, dtype=np.int32)[None], T, F)
    want = T.view(np.uint32)[0] if n >= 5 else T.view(np.uint32)[0] & np.uint32((1 << F) - 1)
    assert np.array_equal(y.view(np.uint32)[0, :len(want)], want)
    # width 6 is the restatement that the BinaryLut6 tests pin
    if n == 6:
        idx = synth.wiring(rng, 30, 20, 6); T = tables(rng, 20, 6); xb = synth.bernoulli_bits(rng, 30, 333, 11)
        assert np.array_equal(oracle.binary_lutn_forward(6, xb, idx, T, 333), oracle.binary_lut6_forward(xb, idx, T, 333))


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is built only where the reference tree is present")
@pytest.mark.parametrize("n", [2, 3, 4, 5, 6])
def test_against_the_compiled_reference(n):
    rng = np.random.default_rng(int.from_bytes(os.urandom(4), "little"))
    for (I, O, F) in [(20, 16, 90), (64, 33, 257)]:
        idx = synth.wiring(rng, I, O, n); T = tables(rng, O, n)
        xb = synth.bernoulli_bits(rng, I, F, (F + 31) // 32)
        y_ref = oracle.ref_binary_lutn(n, xb, idx, T, F)
        y = oracle.binary_lutn_forward(n, xb, idx, T, F)
        assert np.array_equal(synth.unpack_bits(y, F), synth.unpack_bits(y_ref, F))
