"""Writes tests/golden/wiring.npz: the wiring (and, for BinaryLutN, the random truth tables) that the reference's own headers
give a 6-input layer from a seed, a policy string and the layer shapes.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_wiring.py``.  The file holds data only.  The draws go through the C++ standard library's
std::shuffle and std::normal_distribution, so the tables are those of the libstdc++ the harness was built with (GCC 11)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# (kind, seed, policy, input shape, output shape); kind 0 = connection table of StochasticLutN / DifferentiableLutN, 2 = BinaryLutN
CASES = [
    (0, 1, "", [784], [1024]), (0, 7, "random", [20], [64]), (0, 2, "random", [4], [3]), (0, 3, "serial", [10], [7]),
    (0, 5, "pointwise", [8, 5, 4], [12, 5, 4]), (0, 9, "depthwise", [3, 6, 7], [3, 4, 5]), (0, 11, "gauss", [4, 9, 9], [6, 5, 5]),
    (0, 13, "gauss", [100], [30]), (0, 17, "pointwise", [27, 10, 10], [36, 10, 10]),
    (2, 1, "", [100], [50]), (2, 4, "pointwise", [5, 4, 8], [5, 4, 12]), (2, 6, "depthwise", [6, 7, 3], [4, 5, 3]),
    (2, 8, "gauss", [9, 9, 4], [5, 5, 6]), (2, 21, "serial", [12], [5]),
]


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"count": np.array([len(CASES)], np.int32)}
    for k, (kind, seed, policy, ins, outs) in enumerate(CASES):
        p = "c%d_" % k
        out[p + "meta"] = np.array([kind, seed, len(ins)] + ins + outs, np.int64)
        out[p + "policy"] = np.frombuffer(policy.encode(), np.uint8).copy()
        if kind == 0:
            out[p + "idx"] = oracle.ref_wiring6(0, ins, outs, seed, policy)
        else:
            out[p + "idx"], out[p + "table"] = oracle.ref_wiring6(1, ins, outs, seed, policy)
    # a whole StochasticLutN created with a seed (the layer's generator seeds the table)
    idx = np.zeros((64, 6), np.int32)
    import ctypes as C
    f = oracle.ref().bbref_DefaultWiring6
    f.restype = C.c_int
    f(C.c_int(50), C.c_int(64), C.c_uint64(33), idx.ctypes.data_as(C.c_void_p))
    out["layer_idx"] = idx
    out["layer_meta"] = np.array([50, 64, 33], np.int64)
    np.savez_compressed(os.path.join(OUT, "wiring.npz"), **out)
    print("wrote wiring.npz with %d cases" % len(CASES))


if __name__ == "__main__":
    main()
