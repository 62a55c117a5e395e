"""Writes tests/golden/modulation.npz: inputs and outputs of the reference's own RealToBinary, BinaryToReal, Binarize and HardTanh host
classes (include/bb/RealToBinary.h:266-344, BinaryToReal.h:205-352, Binarize.h:142-285, HardTanh.h:133-271), run through
oracle/_ref/libbbref.so, with the objects they serialize to, and BinaryModulation objects (include/bb/BinaryModulation.h:370-394) around
two DifferentiableLut6 layers, and DifferentiableLutDiscrete6 objects (include/bb/DifferentiableLutDiscreteN.h:392-407), whose LUT layers the
reference wired and initialised from a seed.

RealToBinary cases come in two kinds.  "dyadic": inputs on a grid of 1/256 with the range [0, 1] and modulation sizes that are powers
of two, so that every operation of the layer is exact and the reference's build flags (which fuse some multiply-add pairs) cannot
matter: these pin indexing and order bit for bit.  "general": any input, range and sizes; the reference's values are recorded as its
build produced them.  Bits past the last frame of a packed row are not written by the reference and are cleared here.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so`` (``make -C oracle ref``):
``python tests/golden/make_golden_modulation.py``.  The file holds data only."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth           # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))

# depth, points, frames, frame modulation, depth modulation, lo, hi, dyadic, name
REAL_TO_BINARY = [(1, 28, 9, 8, 1, 0.0, 1.0, True, ""), (3, 5, 17, 4, 2, 0.0, 1.0, True, "mod"), (2, 3, 33, 1, 4, 0.0, 1.0, True, ""),
                  (3, 16, 6, 7, 1, 0.0, 1.0, False, ""), (2, 3, 33, 3, 4, -1.0, 2.0, False, ""), (4, 2, 5, 15, 2, 0.1, 0.9, False, "r2b"),
                  (3, 3, 40, 2, 3, 0.0, 255.0, False, "")]
# input nodes, output nodes, output frames, frame mux, name
BINARY_TO_REAL = [(10, 10, 16, 1, ""), (70, 10, 9, 7, ""), (12, 3, 40, 15, "b2r"), (8, 8, 33, 3, ""), (6, 1, 5, 2, "")]
# kind, nodes, frames, th, low, high, window lo, window hi, name
ACTIVATION = [("binarize", 5, 33, 0.0, -1.0, 1.0, -1.0, 1.0, ""), ("binarize", 3, 64, 0.1, 0.0, 1.0, -0.7, 0.9, "bin"),
              ("hard_tanh", 7, 100, 0.0, -1.0, 1.0, -1.0, 1.0, ""), ("hard_tanh", 4, 31, 0.0, -1.0, 1.0, 0.0, 1.0, "ht"),
              ("hard_tanh_binary", 6, 70, 0.0, -1.0, 1.0, -0.5, 0.75, "")]
# BinaryModulation around two DifferentiableLut6 layers: bit activations, input nodes, o1, o2, training modulation, inference
# modulation, depth modulation, seed, dumped after an inference pass, name
MODULATION = [(False, 20, 36, 12, 7, 0, 1, 3, False, ""), (False, 12, 24, 6, 3, 15, 2, 5, True, "net"), (True, 20, 36, 12, 7, 0, 1, 3, False, ""),
              (True, 16, 30, 10, 1, 4, 1, 8, True, "bits")]
# DifferentiableLutDiscrete6 (StochasticLut6 -> StochasticBatchNormalization -> HardTanh): bit activations, input nodes, output nodes,
# seed, batch normalisation, memory saving, name
DISCRETE = [(False, 24, 16, 2, True, False, ""), (False, 12, 40, 6, False, True, "plain"), (True, 24, 16, 2, True, True, "packed"),
            (True, 30, 7, 9, True, False, "")]


def clear_tail(words, frames):
    return synth.pack_bits(synth.unpack_bits(words, frames), words.shape[1])


def main():
    assert oracle.have_ref(), "oracle/_ref/libbbref.so is missing: make -C oracle ref"
    out = {"r2b_count": np.array([len(REAL_TO_BINARY)], np.int32), "b2r_count": np.array([len(BINARY_TO_REAL)], np.int32),
           "act_count": np.array([len(ACTIVATION)], np.int32)}
    for k, (d, p, F, fm, dm, lo, hi, dyadic, name) in enumerate(REAL_TO_BINARY):
        rng = np.random.default_rng(500 + k)
        q = "m%d_" % k
        if dyadic:
            x = (rng.integers(-8, 265, (d * p, F)) / 256.0).astype(np.float32)
        else:
            x = (rng.random((d * p, F)) * (hi - lo) * 1.2 + lo - 0.1 * (hi - lo)).astype(np.float32)
        out[q + "geom"] = np.array([d, p, F, fm, dm, int(dyadic)], np.int64)
        out[q + "range"] = np.array([lo, hi], np.float32)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        out[q + "x"] = x
        out[q + "y_binary"], out[q + "object"] = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, True, name=name, want_object=True)
        yb, out[q + "object_bit"] = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, True, bit=True, name=name, want_object=True)
        out[q + "y_binary_bits"] = clear_tail(yb, F * fm)
        if dm > 1:          # in real mode a layer without depth modulation hands its input through
            out[q + "y_real"], _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, False)
            yb, _ = oracle.ref_real_to_binary(x, d, p, F, fm, dm, lo, hi, False, bit=True)
            out[q + "y_real_bits"] = clear_tail(yb, F * fm)
    for k, (I, O, Fy, fm, name) in enumerate(BINARY_TO_REAL):
        rng = np.random.default_rng(600 + k)
        q = "b%d_" % k
        F = Fy * fm
        x = rng.standard_normal((I, F)).astype(np.float32)
        x[rng.random((I, F)) < 0.1] = 0.0
        xbits = synth.bernoulli_bits(rng, I, F)
        dy = rng.standard_normal((O, Fy)).astype(np.float32)
        y, dx, obj = oracle.ref_binary_to_real(x, O, F, fm, dy=dy, name=name, want_object=True)
        yb, dxb, objb = oracle.ref_binary_to_real(xbits, O, F, fm, bit=True, dy=dy, name=name, want_object=True)
        assert np.array_equal(dx, dxb)
        out[q + "geom"] = np.array([I, O, Fy, fm], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("xbits", xbits), ("dy", dy), ("y", y), ("y_from_bits", yb), ("dx", dx), ("object", obj), ("object_bit", objb)):
            out[q + key] = val
    for k, (kind, nodes, F, th, low, high, lo, hi, name) in enumerate(ACTIVATION):
        rng = np.random.default_rng(700 + k)
        q = "a%d_" % k
        x = rng.standard_normal((nodes, F)).astype(np.float32)
        x[0, :6] = [lo, hi, th, 0.0, -0.0, 0.5]
        dy = rng.standard_normal((nodes, F)).astype(np.float32)
        y, dx, obj = oracle.ref_activation(kind, x, F, th=th, low=low, high=high, lo=lo, hi=hi, dy=dy, name=name, want_object=True)
        yb, dxb, objb = oracle.ref_activation(kind, x, F, bit=True, th=th, low=low, high=high, lo=lo, hi=hi, dy=dy, name=name, want_object=True)
        assert np.array_equal(dx, dxb)
        out[q + "kind"] = np.frombuffer(kind.encode(), np.uint8)
        out[q + "geom"] = np.array([nodes, F], np.int64)
        out[q + "params"] = np.array([th, low, high, lo, hi], np.float32)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        for key, val in (("x", x), ("dy", dy), ("y", y), ("y_bits", clear_tail(yb, F)), ("dx", dx), ("object", obj), ("object_bit", objb)):
            out[q + key] = val
    out["mod_count"] = np.array([len(MODULATION)], np.int32)
    for k, (bit, I, o1, o2, tm, im, dm, seed, infer, name) in enumerate(MODULATION):
        q = "n%d_" % k
        out[q + "args"] = np.array([int(bit), I, o1, o2, tm, im, dm, seed, int(infer)], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        out[q + "object"] = oracle.ref_dump_binary_modulation_object(I, o1, o2, tm, im, dm, bit=bit, seed=seed, run_inference=infer, name=name)
    out["discrete_count"] = np.array([len(DISCRETE)], np.int32)
    for k, (bit, I, O, seed, bn, saving, name) in enumerate(DISCRETE):
        q = "d%d_" % k
        out[q + "args"] = np.array([int(bit), I, O, seed, int(bn), int(saving)], np.int64)
        out[q + "name"] = np.frombuffer(name.encode(), np.uint8)
        out[q + "object"] = oracle.ref_dump_discrete_lut_object(I, O, bit=bit, seed=seed, batch_norm=bn, memory_saving=saving, name=name)
    np.savez_compressed(os.path.join(OUT, "modulation.npz"), **out)
    print("wrote modulation.npz")


if __name__ == "__main__":
    main()
