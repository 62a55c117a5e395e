"""Writes tests/golden/average_lut_objects.npz: AverageLut layers serialized by the reference's own DumpObject
(include/bb/AverageLut.h:412-458), fp32 and bit, through oracle/_ref/libbbref.so.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_average_lut_objects.py``.  The file holds data only: per case the argument list and the bytes."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# n, input nodes, output nodes, bit, binarize_input, binarize_output, name
CASES = [
    (7, 70, 10, False, False, True, ""),
    (7, 70, 10, True, False, True, "vote"),
    (3, 12, 5, False, True, False, "sum"),
    (16, 64, 2, True, True, True, ""),
]


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"count": np.array([len(CASES)], np.int32)}
    for k, (n, I, O, bit, bin_in, bin_out, name) in enumerate(CASES):
        rng = np.random.default_rng(200 + k)
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        p = "a%d_" % k
        out[p + "args"] = np.array([n, I, O, int(bit), int(bin_in), int(bin_out)], np.int64)
        out[p + "name"] = np.frombuffer(name.encode(), np.uint8)
        out[p + "idx"] = idx
        out[p + "bytes"] = oracle.ref_average_lut_object(idx, I, bit, bin_in, bin_out, name)
    np.savez_compressed(os.path.join(OUT, "average_lut_objects.npz"), **out)
    print("wrote average_lut_objects.npz:", len(CASES), "cases")


if __name__ == "__main__":
    main()
