"""Writes tests/golden/container_objects.npz: serialized container objects as the reference's own DumpObject writes them — the
convolution wrapper (include/bb/Convolution2d.h:355-409) around one DifferentiableLut6 layer and around a list of two, the list
alone (include/bb/Sequential.h:239-288), ConvolutionIm2Col (:492-563) and ConvolutionCol2Im (:334-367).

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_containers.py``.  The file holds data only: each case is the argument list it was made from and
the bytes.  The LUT layers inside are wired and initialised by the reference from the seed; the tests only need their bytes to
survive a load and a dump."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# kind (0 conv over one layer, 1 conv over a list of two, 2 the list, 3 Im2Col, 4 Col2Im), c, h, w, fh, fw, ys, xs, same, border, o1, o2, seed, name
CASES = [
    (0, 3, 8, 9, 3, 3, 1, 1, False, "reflect_101", 0, 12, 5, ""),
    (0, 2, 7, 7, 3, 3, 2, 2, True, "constant", 0, 8, 9, "conv_a"),
    (1, 3, 8, 8, 3, 3, 1, 1, False, "reflect_101", 24, 12, 3, ""),
    (1, 1, 6, 10, 2, 3, 1, 2, True, "wrap", 16, 7, 11, "conv_b"),
    (2, 3, 1, 1, 3, 3, 1, 1, False, "reflect_101", 30, 10, 2, "body"),
    (2, 2, 1, 1, 2, 2, 1, 1, False, "reflect_101", 12, 6, 4, ""),
    (3, 3, 32, 32, 3, 3, 1, 1, False, "reflect_101", 0, 0, 0, ""),
    (3, 4, 9, 7, 5, 3, 2, 1, True, "replicate", 0, 0, 0, "taps"),
    (4, 0, 30, 30, 1, 1, 1, 1, False, "reflect_101", 0, 36, 0, ""),
    (4, 0, 5, 4, 1, 1, 1, 1, False, "reflect_101", 0, 7, 0, "images"),
]


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"count": np.array([len(CASES)], np.int32)}
    for k, (kind, c, h, w, fh, fw, ys, xs, same, border, o1, o2, seed, name) in enumerate(CASES):
        p = "c%d_" % k
        out[p + "args"] = np.array([kind, c, h, w, fh, fw, ys, xs, int(same), o1, o2, seed], np.int64)
        out[p + "border"] = np.frombuffer(border.encode(), np.uint8).copy()
        out[p + "name"] = np.frombuffer(name.encode(), np.uint8).copy()
        out[p + "bytes"] = oracle.ref_dump_container_object(kind, c, h, w, fh, fw, ys, xs, same, border, o1, o2, seed, name)
    np.savez_compressed(os.path.join(OUT, "container_objects.npz"), **out)
    print("wrote container_objects.npz:", len(CASES), "objects,", sum(int(out["c%d_bytes" % k].size) for k in range(len(CASES))), "bytes")


if __name__ == "__main__":
    main()
