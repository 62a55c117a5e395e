"""Writes tests/golden/pooling.npz: inputs and outputs of the reference's own MaxPooling, UpSampling and Shuffle host classes
(include/bb/MaxPooling.h:192-579, include/bb/UpSampling.h:168-353, include/bb/Shuffle.h:146-249), fp32 and packed bits, run through oracle/_ref/libbbref.so, with
the objects they serialize to.  Bits past the last frame of a packed row are not defined by the reference and are cleared here.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_pooling.py``.  The file holds data only."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth           # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# channels, height, width, filter height, filter width, frames, name
POOL = [(3, 4, 6, 2, 3, 2, ""), (2, 5, 7, 2, 2, 33, "pool"), (1, 8, 8, 3, 3, 64, ""), (4, 3, 3, 1, 1, 5, ""), (2, 6, 5, 2, 4, 40, ""),
        (6, 30, 30, 2, 2, 2, "cifar")]
# channels, height, width, filter height, filter width, fill, frames, name
UP = [(3, 2, 3, 2, 2, True, 7, ""), (2, 4, 3, 3, 2, False, 33, "up"), (1, 5, 5, 1, 1, True, 64, ""), (4, 3, 2, 2, 3, True, 40, ""),
      (2, 3, 3, 2, 2, False, 5, "")]
# nodes, shuffle unit, frames, name
SHUFFLE = [(6, 3, 2, ""), (84, 7, 33, "deal"), (64, 1, 5, ""), (64, 64, 40, ""), (30, 5, 70, "")]


def clear_tail(words, frames):
    return synth.pack_bits(synth.unpack_bits(words, frames), words.shape[1])


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"pool_count": np.array([len(POOL)], np.int32), "up_count": np.array([len(UP)], np.int32),
           "shuffle_count": np.array([len(SHUFFLE)], np.int32)}
    for k, (c, h, w, fh, fw, F, name) in enumerate(POOL):
        rng = np.random.default_rng(800 + k)
        q = "p%d_" % k
        x = rng.standard_normal((c * h * w, F)).astype(np.float32)
        x[rng.random(x.shape) < 0.2] = 0.5                                      # ties: the first largest value wins
        xbits = synth.bernoulli_bits(rng, c * h * w, F, p=0.3)
        O = c * ((h + fh - 1) // fh) * ((w + fw - 1) // fw)
        dy = rng.standard_normal((O, F)).astype(np.float32)
        y, dx, obj = oracle.ref_max_pooling(x, c, h, w, fh, fw, F, dy=dy, name=name, want_object=True)
        yb, dxb, objb = oracle.ref_max_pooling(xbits, c, h, w, fh, fw, F, bit=True, dy=dy, name=name, want_object=True)
        out[q + "geom"] = np.array([c, h, w, fh, fw, F], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("xbits", xbits), ("dy", dy), ("y", y), ("dx", dx), ("y_bits", clear_tail(yb, F)), ("dx_from_bits", dxb),
                         ("object", obj), ("object_bit", objb)):
            out[q + key] = val
    for k, (c, h, w, fh, fw, fill, F, name) in enumerate(UP):
        rng = np.random.default_rng(900 + k)
        q = "u%d_" % k
        x = rng.standard_normal((c * h * w, F)).astype(np.float32)
        xbits = synth.bernoulli_bits(rng, c * h * w, F)
        dy = rng.standard_normal((c * h * fh * w * fw, F)).astype(np.float32)
        y, dx, obj = oracle.ref_up_sampling(x, c, h, w, fh, fw, F, fill, dy=dy, name=name, want_object=True)
        yb, _, objb = oracle.ref_up_sampling(xbits, c, h, w, fh, fw, F, fill, bit=True, name=name, want_object=True)
        out[q + "geom"] = np.array([c, h, w, fh, fw, int(fill), F], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("xbits", xbits), ("dy", dy), ("y", y), ("dx", dx), ("y_bits", clear_tail(yb, F)), ("object", obj), ("object_bit", objb)):
            out[q + key] = val
    for k, (nodes, unit, F, name) in enumerate(SHUFFLE):
        rng = np.random.default_rng(1000 + k)
        q = "s%d_" % k
        x = rng.standard_normal((nodes, F)).astype(np.float32)
        xbits = synth.bernoulli_bits(rng, nodes, F)
        dy = rng.standard_normal((nodes, F)).astype(np.float32)
        dybits = synth.bernoulli_bits(rng, nodes, F)
        y, dx, obj = oracle.ref_shuffle(x, unit, F, dy=dy, name=name, want_object=True)
        yb, dxb, _ = oracle.ref_shuffle(xbits, unit, F, bit=True, dy=dybits)
        out[q + "geom"] = np.array([nodes, unit, F], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("xbits", xbits), ("dy", dy), ("dybits", dybits), ("y", y), ("dx", dx), ("y_bits", clear_tail(yb, F)),
                         ("dx_bits", clear_tail(dxb, F)), ("object", obj)):
            out[q + key] = val
    np.savez_compressed(os.path.join(OUT, "pooling.npz"), **out)
    print("wrote pooling.npz")


if __name__ == "__main__":
    main()
