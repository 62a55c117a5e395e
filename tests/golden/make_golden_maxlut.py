"""Writes tests/golden/maxlut.npz: inputs and outputs of the reference's own MaxLut host class (include/bb/MaxLut.h: forward
:293-318, backward :394-424, serialization :428-465), run through oracle/_ref/libbbref.so.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_maxlut.py``.  The file holds data only.  The reference's backward loop adds into shared rows
from an OpenMP loop over nodes without synchronisation; it is run with one thread, which is the loop's serial meaning."""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth           # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# n, input nodes, output nodes, frames, binarize_output, name
CASES = [
    (6, 12, 2, 3, True, ""),
    (6, 40, 16, 70, True, "pool"),
    (6, 40, 16, 70, False, ""),
    (3, 9, 20, 33, False, ""),
    (9, 30, 5, 129, True, "wide"),
    (1, 4, 4, 10, False, ""),
]


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    ctypes.CDLL("libgomp.so.1").omp_set_num_threads(1)
    out = {"count": np.array([len(CASES)], np.int32)}
    for k, (n, I, O, F, bin_out, name) in enumerate(CASES):
        rng = np.random.default_rng(100 + k)
        p = "m%d_" % k
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        x = (rng.random((I, F)) * 3 - 2).astype(np.float32)            # in [-2, 1): some nodes see nothing above -1
        x[rng.random(x.shape) < 0.1] = 0.0
        x[:, ::7] = np.round(x[:, ::7])                                 # ties between inputs
        dy = rng.standard_normal((O, F)).astype(np.float32)
        xbits = synth.bernoulli_bits(rng, I, F, p=0.2)
        y, dx, obj = oracle.ref_max_lut(x, idx, I, F, binarize_output=bin_out, dy=dy, name=name, want_object=True)
        yb, dxb, objb = oracle.ref_max_lut(xbits, idx, I, F, bit=True, dy=dy, name=name, want_object=True)
        out[p + "geom"] = np.array([n, I, O, F, int(bin_out)], np.int64)
        out[p + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("idx", idx), ("x", x), ("dy", dy), ("xbits", xbits), ("y", y), ("dx", dx), ("ybits", yb), ("dxbits", dxb),
                         ("object", obj), ("object_bit", objb)):
            out[p + key] = val
    np.savez_compressed(os.path.join(OUT, "maxlut.npz"), **out)
    print("wrote maxlut.npz:", len(CASES), "cases")


if __name__ == "__main__":
    main()
