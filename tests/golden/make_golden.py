"""Writes tests/golden/*.npz: input/output vectors produced by the reference's own CPU headers.

Run in a container that holds the reference tree and a built ``oracle/_ref/libbbref.so``
(``make -C oracle ref``):  ``python tests/golden/make_golden.py``.
The files hold data only (inputs, flags and the arrays the reference returned); padding bits of packed outputs
are masked to zero because the reference leaves them undefined.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                               # noqa: E402
from binarybrain_amd import synth          # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def mask_bits(packed, frames):
    return synth.pack_bits(synth.unpack_bits(packed, frames), packed.shape[1])


def stochastic_cases():
    rng = np.random.default_rng(20240601)
    cases = {}
    k = 0
    for (n, I, O, F, simd) in [(6, 32, 16, 64, 1), (6, 14, 16, 8, 1), (6, 13, 17, 29, 0), (4, 20, 16, 40, 0), (2, 9, 8, 24, 0)]:
        for (binary_mode, lut_binarize) in [(0, 0), (0, 1), (1, 0)]:
            idx = synth.wiring(rng, I, O, n)
            W = synth.lut_tables(rng, O, n, -0.1, 1.1)
            x = synth.uniform_frames(rng, I, F, stride=F, lo=-0.1, hi=1.1)
            dy = synth.normal_frames(rng, O, F, stride=F)
            dW0 = rng.standard_normal((O, 1 << n)).astype(np.float32)
            r = oracle.ref_stochastic_lut(n, x, idx, W, dy=dy, dW_init=dW0, binary_mode=binary_mode,
                                          lut_binarize=lut_binarize, host_simd=simd)
            p = "c%d_" % k
            cases.update({p + "meta": np.array([n, I, O, F, simd, binary_mode, lut_binarize], np.int32),
                          p + "idx": idx, p + "W": W, p + "x": x, p + "dy": dy, p + "dW0": dW0,
                          p + "Wc": r["W"], p + "y": r["y"], p + "dx": r["dx"], p + "dW": r["dW"]})
            k += 1
    # bit-packed input
    for (n, I, O, F) in [(6, 24, 16, 70), (4, 12, 8, 33)]:
        for lut_binarize in (0, 1):
            idx = synth.wiring(rng, I, O, n)
            W = synth.lut_tables(rng, O, n)
            xb = synth.bernoulli_bits(rng, I, F)
            dy = synth.normal_frames(rng, O, F, stride=F)
            r = oracle.ref_stochastic_lut(n, xb, idx, W, dy=dy, bit_input=True, lut_binarize=lut_binarize, frame_size=F)
            p = "c%d_" % k
            cases.update({p + "meta": np.array([n, I, O, F, -1, 1, lut_binarize], np.int32),
                          p + "idx": idx, p + "W": W, p + "xbits": xb, p + "dy": dy,
                          p + "Wc": r["W"], p + "y": r["y"], p + "dx": r["dx"], p + "dW": r["dW"]})
            k += 1
    cases["count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "stochastic_lut.npz"), **cases)


def differentiable_cases():
    rng = np.random.default_rng(20240602)
    cases = {}
    k = 0
    for (n, I, O, F) in [(6, 20, 16, 40), (6, 16, 8, 131), (4, 20, 16, 39), (2, 10, 8, 64)]:
        for (bit, binary_mode, lut_binarize, batch_norm) in [(0, 1, 0, 1), (0, 0, 0, 1), (0, 1, 1, 1), (1, 1, 0, 1),
                                                              (0, 1, 0, 0), (0, 0, 0, 0), (1, 1, 0, 0)]:
            idx = synth.wiring(rng, I, O, n)
            W = synth.lut_tables(rng, O, n)
            dy = synth.normal_frames(rng, O, F, stride=F)
            rm = rng.random(O).astype(np.float32)
            rv = (rng.random(O) + 0.5).astype(np.float32)
            x = synth.bernoulli_bits(rng, I, F) if bit else synth.uniform_frames(rng, I, F, stride=F, lo=-0.1, hi=1.1)
            kw = dict(bit_input=bool(bit), batch_norm=bool(batch_norm), binary_mode=bool(binary_mode),
                      lut_binarize=bool(lut_binarize), frame_size=F, gamma=0.3, beta=0.5, momentum=0.9)
            r = oracle.ref_differentiable_lut(n, x, idx, W, rm, rv, dy=dy, train=True, **kw)
            ri = oracle.ref_differentiable_lut(n, x, idx, W, rm, rv, train=False, **kw)
            y, yi = r["y"], ri["y"]
            if bit:
                y, yi = mask_bits(y, F), mask_bits(yi, F)
            p = "c%d_" % k
            cases.update({p + "meta": np.array([n, I, O, F, bit, binary_mode, lut_binarize, batch_norm], np.int32),
                          p + "idx": idx, p + "W": W, p + "x": x, p + "dy": dy, p + "rm": rm, p + "rv": rv,
                          p + "y": y, p + "y_inf": yi, p + "dx": r["dx"], p + "dW": r["dW"],
                          p + "mean": r["mean"], p + "rstd": r["rstd"],
                          p + "rm_out": r["running_mean"], p + "rv_out": r["running_var"]})
            k += 1
    cases["count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "differentiable_lut.npz"), **cases)


def binary_cases():
    rng = np.random.default_rng(20240603)
    cases = {}
    k = 0
    for (I, O, F) in [(16, 16, 32), (64, 32, 512), (70, 33, 1000), (8, 5, 7)]:
        idx = synth.wiring(rng, I, O, 6)
        T = synth.truth_tables(rng, O)
        xb = synth.bernoulli_bits(rng, I, F)
        y_simd = mask_bits(oracle.ref_binary_lut6(xb, idx, T, F, host_simd=True), F)
        y_gen = mask_bits(oracle.ref_binary_lut6(xb, idx, T, F, host_simd=False), F)
        assert np.array_equal(y_simd, y_gen)
        rev = oracle.ref_reverse_table6(idx, I)
        p = "c%d_" % k
        cases.update({p + "meta": np.array([I, O, F], np.int32), p + "idx": idx, p + "table": T, p + "xbits": xb,
                      p + "y": y_simd, p + "rev": rev})
        k += 1
    cases["count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "binary_lut6.npz"), **cases)


def adam_cases():
    """bb::OptimizerAdam<float> and the elementwise Tensor kernels of the reference (host path)."""
    rng = np.random.default_rng(20240604)
    cases = {}
    k = 0
    for (size, steps, lr, b1, b2) in [(1, 10, 0.001, 0.9, 0.999), (257, 12, 0.001, 0.9, 0.999), (64, 5, 0.01, 0.8, 0.99)]:
        p0 = rng.standard_normal(size).astype(np.float32)
        g = (rng.standard_normal((steps, size)) * 2.0 + 0.0001).astype(np.float32)
        if size > 8:
            g[:, 3] = 0.0                                   # a parameter that never receives a gradient
        p1 = oracle.ref_adam_steps(p0, list(g), lr, b1, b2)
        q = "a%d_" % k
        cases.update({q + "hyper": np.array([lr, b1, b2], np.float64), q + "p0": p0, q + "g": g, q + "p": p1})
        k += 1
    cases["adam_count"] = np.array([k], np.int32)
    x = (rng.standard_normal(301) * 3.0).astype(np.float32)
    y = (rng.standard_normal(301) * 3.0).astype(np.float32)
    pos = np.abs(x) + np.float32(0.01)
    cases.update({"vx": x, "vy": y, "vpos": pos, "coef": np.array([1.5, -0.75, 0.25, 2.0], np.float32)})
    a, b, c, d = [float(v) for v in cases["coef"]]
    cases["add_ex"] = oracle.ref_vector_op("add_ex", x, y, a, b, c)
    cases["mul_ex"] = oracle.ref_vector_op("mul_ex", x, y, a, b)
    cases["div_ex"] = oracle.ref_vector_op("div_ex", x, pos, a, b, c, d)
    cases["sqrt"] = oracle.ref_vector_op("sqrt", pos)
    cases["exp"] = oracle.ref_vector_op("exp", x)
    cases["min"] = oracle.ref_vector_op("min", x, y)
    cases["min_v"] = oracle.ref_vector_op("min_v", x, None, 0.3)
    cases["max"] = oracle.ref_vector_op("max", x, y)
    cases["max_v"] = oracle.ref_vector_op("max_v", x, None, 0.3)
    np.savez_compressed(os.path.join(OUT, "adam.npz"), **cases)


def conv_cases():
    """ConvolutionIm2Col, ConvolutionCol2Im and StochasticMaxPooling2x2 of the reference (host paths)."""
    rng = np.random.default_rng(20240605)
    cases = {}
    k = 0
    for (c, h, w, F, fh, fw, ys, xs, pad, border) in [(2, 3, 4, 2, 2, 3, 1, 1, "valid", "reflect_101"),
                                                      (3, 7, 6, 5, 3, 3, 1, 1, "same", "reflect_101"),
                                                      (2, 8, 9, 3, 3, 3, 2, 2, "same", "replicate"),
                                                      (1, 5, 5, 4, 3, 3, 2, 1, "valid", "constant"),
                                                      (2, 6, 7, 3, 3, 5, 1, 1, "same", "wrap"),
                                                      (2, 6, 7, 35, 3, 3, 1, 1, "same", "reflect"),
                                                      (3, 9, 8, 3, 3, 3, 1, 2, "same", "constant")]:
        x = rng.random((c * h * w, F)).astype(np.float32)
        oh, ow, _, _ = oracle.im2col_geometry(h, w, fh, fw, ys, xs, pad)
        dy = rng.standard_normal((c * fh * fw, F * oh * ow)).astype(np.float32)
        y, dx = oracle.ref_im2col(x, c, h, w, F, fh, fw, ys, xs, pad, border, dy=dy)
        xb = synth.bernoulli_bits(rng, c * h * w, F)
        yb, _ = oracle.ref_im2col(xb, c, h, w, F, fh, fw, ys, xs, pad, border, bit=True)
        q = "i%d_" % k
        cases.update({q + "geom": np.array([c, h, w, F, fh, fw, ys, xs, int(pad == "same"), oracle.BORDER_MODES[border]], np.int32),
                      q + "x": x, q + "dy": dy, q + "y": y, q + "dx": dx, q + "xbits": xb, q + "ybits": mask_bits(yb, F * oh * ow)})
        k += 1
    cases["im2col_count"] = np.array([k], np.int32)
    k = 0
    for (c, h, w, F) in [(3, 4, 5, 6), (2, 1, 7, 33), (5, 3, 3, 64)]:
        x = rng.random((c, F * h * w)).astype(np.float32)
        dy = rng.standard_normal((c * h * w, F)).astype(np.float32)
        y, dx = oracle.ref_col2im(x, c, h, w, F, dy=dy)
        xb = synth.bernoulli_bits(rng, c, F * h * w)
        yb, _ = oracle.ref_col2im(xb, c, h, w, F, bit=True)
        q = "c%d_" % k
        cases.update({q + "geom": np.array([c, h, w, F], np.int32), q + "x": x, q + "dy": dy, q + "y": y, q + "dx": dx,
                      q + "xbits": xb, q + "ybits": mask_bits(yb, F)})
        k += 1
    cases["col2im_count"] = np.array([k], np.int32)
    k = 0
    for (c, h, w, F) in [(2, 4, 6, 5), (3, 5, 7, 9), (1, 1, 1, 3), (2, 30, 30, 16)]:
        x = rng.random((c * h * w, F)).astype(np.float32)
        dy = rng.standard_normal((c * ((h + 1) // 2) * ((w + 1) // 2), F)).astype(np.float32)
        y, dx = oracle.ref_stochastic_maxpool2x2(x, c, h, w, F, dy=dy)
        q = "p%d_" % k
        cases.update({q + "geom": np.array([c, h, w, F], np.int32), q + "x": x, q + "dy": dy, q + "y": y, q + "dx": dx})
        k += 1
    cases["pool_count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "conv.npz"), **cases)


def tail_cases():
    """AverageLut, LossSoftmaxCrossEntropy and MetricsCategoricalAccuracy of the reference (host paths)."""
    rng = np.random.default_rng(20240611)
    cases = {}
    k = 0
    # AverageLut::Backward runs `#pragma omp parallel for` over output nodes around an unsynchronised dx += (AverageLut.h:395-404):
    # with several threads, nodes that share an input lose updates.  One thread gives the loop its serial meaning.
    import ctypes
    gomp = ctypes.CDLL("libgomp.so.1")
    threads = gomp.omp_get_max_threads()
    gomp.omp_set_num_threads(1)
    for (n, I, O, F, bin_in, bin_out) in [(7, 70, 10, 37, False, True), (7, 70, 10, 37, False, False), (4, 9, 5, 64, True, True),
                                          (6, 12, 16, 33, True, False), (1, 3, 3, 5, False, False), (8, 8, 2, 100, False, True)]:
        idx = rng.integers(0, I, (O, n)).astype(np.int32)              # repeats allowed: AverageLut wiring need not be distinct
        x = (rng.random((I, F)) * 2 - 1).astype(np.float32)
        x[rng.random((I, F)) < 0.1] = 0.0                               # exact zeros sit on the binarize threshold
        dy = rng.standard_normal((O, F)).astype(np.float32)
        y, dx = oracle.ref_average_lut(x, idx, I, F, binarize_input=bin_in, binarize_output=bin_out, dy=dy)
        xb = synth.bernoulli_bits(rng, I, F)
        yb, _ = oracle.ref_average_lut(xb, idx, I, F, bit=True, binarize_input=bin_in, binarize_output=bin_out)
        q = "a%d_" % k
        cases.update({q + "geom": np.array([n, I, O, F, int(bin_in), int(bin_out)], np.int32), q + "idx": idx, q + "x": x, q + "dy": dy,
                      q + "y": y, q + "dx": dx, q + "xbits": xb, q + "ybits": mask_bits(yb, F)})
        k += 1
    cases["average_count"] = np.array([k], np.int32)
    gomp.omp_set_num_threads(threads)
    k = 0
    for (ch, pix, F, kind) in [(10, 1, 33, "onehot"), (10, 1, 64, "sharp"), (4, 6, 17, "onehot"), (3, 5, 20, "weighted"), (7, 1, 9, "ties")]:
        y = (rng.standard_normal((ch * pix, F)) * (30.0 if kind == "sharp" else 1.0)).astype(np.float32)
        t = np.zeros((ch * pix, F), np.float32)
        for f in range(F):
            for p in range(pix):
                if kind == "weighted" and rng.random() < 0.3:
                    continue                                            # an unlabeled pixel
                c = int(rng.integers(0, ch))
                t[c * pix + p, f] = 1.0 if kind != "weighted" else np.float32(rng.integers(1, 4) * 0.5)
        if kind == "ties":
            y = np.round(y)                                             # repeated maxima: the first channel decides
        dy, loss, metric = oracle.ref_loss_and_accuracy(y, t, ch, pix, F)
        q = "l%d_" % k
        cases.update({q + "geom": np.array([ch, pix, F], np.int32), q + "y": y, q + "t": t, q + "dy": dy,
                      q + "loss": np.array([loss], np.float64), q + "metric": np.array([metric], np.float64)})
        k += 1
    cases["loss_count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "tail.npz"), **cases)


def object_cases():
    """6-input LUT layers serialized by the reference's own Object::DumpObject (`.bb_net` object bytes)."""
    rng = np.random.default_rng(20240617)
    cases = {}
    k = 0
    for (kind, bit, I, O, flags, name) in [("stochastic", 0, 20, 7, 2, ""), ("stochastic", 1, 9, 3, 3, "lut_a"),
                                            ("differentiable", 0, 16, 5, 5, "layer0"), ("differentiable", 1, 12, 4, 7, ""),
                                            ("differentiable", 0, 8, 2, 0, "plain"), ("binary", 1, 33, 11, 0, "packed")]:
        idx = np.stack([rng.choice(I, 6, replace=False) for _ in range(O)]).astype(np.int32)
        params = rng.integers(-2**31, 2**31, (O, 2)).astype(np.int32) if kind == "binary" else rng.random((O, 64)).astype(np.float32)
        mean = rng.random(O).astype(np.float32); var = (rng.random(O) + 0.5).astype(np.float32)
        data = oracle.ref_dump_lut_object(kind, bit, I, idx, params, mean, var, flags, (0.75, 0.4, 0.6), name)
        q = "o%d_" % k
        cases.update({q + "desc": np.array([oracle.LUT_OBJECT_KINDS[kind], bit, I, O, flags], np.int32), q + "name": np.frombuffer(name.encode(), np.uint8),
                      q + "idx": idx, q + "params": params, q + "mean": mean, q + "var": var, q + "bytes": np.frombuffer(data, np.uint8)})
        k += 1
    cases["object_count"] = np.array([k], np.int32)
    np.savez_compressed(os.path.join(OUT, "objects.npz"), **cases)


if __name__ == "__main__":
    assert oracle.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    which = sys.argv[1:] or ["stochastic", "differentiable", "binary", "adam", "conv", "tail", "objects"]
    if "stochastic" in which: stochastic_cases()
    if "differentiable" in which: differentiable_cases()
    if "binary" in which: binary_cases()
    if "adam" in which: adam_cases()
    if "conv" in which: conv_cases()
    if "tail" in which: tail_cases()
    if "objects" in which: object_cases()
    for f in sorted(os.listdir(OUT)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(OUT, f)), "bytes")
