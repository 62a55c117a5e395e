"""Writes tests/golden/bn.npz: inputs and outputs of the reference's own StochasticBatchNormalization<float> host class
(include/bb/StochasticBatchNormalization.h: training forward :535-597, backward :815-851, serialization :143-183), run through
oracle/_ref/libbbref.so.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_bn.py``.  The file holds data only.  Each case: geometry and scalars, x, dy, the running
statistics before and after, y, the batch mean and reciprocal deviation, dx, and the layer's serialized bytes after the pass."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# nodes, frames, momentum, gamma, beta, seed, input kind (0 uniform [0, 1], 1 normal, 2 one constant row among uniform ones), name
CASES = [
    (7, 33, 0.9, 0.2, 0.5, 1, 0, ""),
    (16, 128, 0.9, 0.2, 0.5, 2, 1, "bn0"),
    (5, 1, 0.5, 0.3, 0.4, 3, 0, ""),
    (3, 257, 0.0, 1.0, 0.0, 4, 1, ""),
    (9, 64, 0.99, 0.25, 0.5, 5, 2, "flat_row"),
]


def make_case(nodes, frames, seed, kind):
    rng = np.random.default_rng(seed)
    x = rng.random((nodes, frames)) if kind != 1 else rng.standard_normal((nodes, frames)) * 2 + 0.3
    x = x.astype(np.float32)
    if kind == 2:
        x[nodes // 2, :] = np.float32(0.625)
    dy = rng.standard_normal((nodes, frames)).astype(np.float32)
    rm = rng.standard_normal(nodes).astype(np.float32)
    rv = (rng.random(nodes) + 0.5).astype(np.float32)
    return x, dy, rm, rv


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"count": np.array([len(CASES)], np.int32)}
    for k, (nodes, frames, momentum, gamma, beta, seed, kind, name) in enumerate(CASES):
        p = "b%d_" % k
        x, dy, rm, rv = make_case(nodes, frames, seed, kind)
        r = oracle.ref_stochastic_bn(x, rm, rv, gamma, beta, momentum, train=True, dy=dy, name=name, want_object=True)
        out[p + "geom"] = np.array([nodes, frames], np.int64)
        out[p + "scalars"] = np.array([momentum, gamma, beta], np.float32)
        out[p + "name"] = np.frombuffer(name.encode(), np.uint8)
        out[p + "x"] = x; out[p + "dy"] = dy; out[p + "running_mean_in"] = rm; out[p + "running_var_in"] = rv
        for key in ("y", "mean", "rstd", "running_mean", "running_var", "dx", "object"):
            out[p + key] = r[key]
    np.savez_compressed(os.path.join(OUT, "bn.npz"), **out)
    print("wrote bn.npz:", len(CASES), "cases")


if __name__ == "__main__":
    main()
