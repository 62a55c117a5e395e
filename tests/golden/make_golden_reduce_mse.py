"""Writes tests/golden/reduce_mse.npz: inputs and outputs of the reference's own Reduce, LossMeanSquaredError and
MetricsMeanSquaredError host classes (include/bb/Reduce.h:130-250, LossMeanSquaredError.h:91-171, MetricsMeanSquaredError.h:53-85),
run through oracle/_ref/libbbref.so.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_reduce_mse.py``.  The file holds data only."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth           # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# input nodes, output nodes, frames, integration size (0: output shape given), name
REDUCE = [(70, 10, 33, 0, ""), (70, 10, 33, 7, "fold"), (12, 12, 5, 0, ""), (96, 3, 130, 0, ""), (40, 8, 64, 5, "")]
# nodes, frames per batch, batches, reduction "sum"
MSE = [(10, 37, 1, False), (10, 37, 3, False), (3, 64, 2, True), (1, 5, 1, False), (50, 200, 2, False)]


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"reduce_count": np.array([len(REDUCE)], np.int32), "mse_count": np.array([len(MSE)], np.int32)}
    for k, (I, O, F, integ, name) in enumerate(REDUCE):
        rng = np.random.default_rng(300 + k)
        p = "r%d_" % k
        x = rng.standard_normal((I, F)).astype(np.float32)
        dy = rng.standard_normal((O, F)).astype(np.float32)
        xbits = synth.bernoulli_bits(rng, I, F)
        y, dx, obj = oracle.ref_reduce(x, O, F, integration_size=integ, dy=dy, name=name, want_object=True)
        yb, dxb, objb = oracle.ref_reduce(xbits, O, F, bit=True, integration_size=integ, dy=dy, name=name, want_object=True)
        out[p + "geom"] = np.array([I, O, F, integ], np.int64)
        out[p + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("dy", dy), ("xbits", xbits), ("y", y), ("dx", dx), ("y_from_bits", yb), ("object", obj), ("object_bit", objb)):
            out[p + key] = val
        assert np.array_equal(dx, dxb)
    for k, (nodes, F, batches, rsum) in enumerate(MSE):
        rng = np.random.default_rng(400 + k)
        p = "e%d_" % k
        y = rng.random((nodes, F * batches)).astype(np.float32)
        t = (rng.random((nodes, F * batches)) > 0.5).astype(np.float32)
        dy, loss, metric = oracle.ref_mean_squared_error(y, t, F, batches, rsum)
        out[p + "geom"] = np.array([nodes, F, batches, int(rsum)], np.int64)
        out[p + "y"] = y; out[p + "t"] = t; out[p + "dy"] = dy
        out[p + "loss_metric"] = np.array([loss, metric], np.float64)
    np.savez_compressed(os.path.join(OUT, "reduce_mse.npz"), **out)
    print("wrote reduce_mse.npz")


if __name__ == "__main__":
    main()
