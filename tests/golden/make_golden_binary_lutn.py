"""Writes tests/golden/binary_lutn.npz: BinaryLutN<N, Bit> for N = 2 .. 5 run by the reference's own class (its generic host loop,
include/bb/BinaryLutN.h:436-463) through oracle/_ref.  Run where the reference tree is present and ``make -C oracle ref`` has built
the library:  ``python tests/golden/make_golden_binary_lutn.py``.  Data only: wiring, one table word per node, packed inputs and the
packed outputs the reference returned (bits past the last frame masked to zero: the reference leaves them undefined)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth          # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    assert oracle.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    rng = np.random.default_rng(20261125)
    cases = {}
    k = 0
    for n in (2, 3, 4, 5):
        for (I, O, F) in [(16, 12, 64), (9, 5, 37), (40, 33, 300)]:
            idx = synth.wiring(rng, I, O, n)
            table = rng.integers(0, 1 << (1 << n), (O, 1), dtype=np.int64).astype(np.uint32).view(np.int32)
            xb = synth.bernoulli_bits(rng, I, F, (F + 31) // 32)
            y = oracle.ref_binary_lutn(n, xb, idx, table, F)
            y = synth.pack_bits(synth.unpack_bits(y, F), y.shape[1])
            p = "c%d_" % k
            cases.update({p + "meta": np.array([n, I, O, F], np.int32), p + "idx": idx, p + "table": table, p + "xbits": xb, p + "y": y})
            k += 1
    cases["count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "binary_lutn.npz"), **cases)
    print("binary_lutn.npz: %d cases" % k)


if __name__ == "__main__":
    main()
