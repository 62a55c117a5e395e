"""GPU parity on random shapes: LUT width, node and frame counts, row pitches, input kind (fp32, fp32 binarized, packed
bits), table binarization, batch-norm or not, and the dx mode are drawn from a seeded generator; every case goes through
the C ABI and is compared with the CPU oracle at the tolerances of the other GPU tests (BinaryLut6, the bit-to-bit forward,
Im2Col, Col2Im and pooling, drawn the same way, bit for bit; AverageLut, the loss, accuracy and Adam at their own tests' bars).  What the draws hit that fixed
cases rarely do, and how the comparison deals with it:
  * a table that is constant after binarization has dx = 0 exactly, and batch-norm can cancel a whole table gradient: the
    oracle then holds rounding noise, so dx and dW are measured against max(|reference|, |dy|);
  * the oracle's var = E[y^2] - E[y]^2 (the reference's formula) loses digits when var is small against mean^2 (narrow
    LUTs on two-valued inputs): rstd gets 1e-7 / var on top of its 1e-4;
  * frames whose batch-norm output is within 1e-5 of the binarization threshold or of an edge of the hard-tanh window may
    fall on either side (sometimes for a whole class of frames, when a corner value of a binarized table equals the
    mean): outputs are compared away from the threshold, and dy is zeroed at the window's edges."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from test_gpu_differentiable_lut import _pre_activation
from util import dev, host

pytestmark = pytest.mark.gpu


def rel_err(a, b, floor=0.0):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), floor, 1e-30))


def stride_fp32(rng, F):
    return int(rng.choice([F, ((F + 63) // 64) * 64, synth.frame_stride_fp32(F), F + int(rng.integers(0, 70))]))


def run_case(ops, torch, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.choice([2, 3, 4, 5, 6], p=[0.1, 0.1, 0.15, 0.15, 0.5]))
    I = int(rng.integers(n, 300)); O = int(rng.integers(1, 200))
    F = int(rng.choice([int(rng.integers(1, 70)), int(rng.integers(64, 700)), int(rng.integers(700, 5000))]))
    kind = str(rng.choice(["st_fp32", "st_bin", "st_bit", "dl_fp32", "dl_bit"]))
    lut_binarize = int(rng.integers(0, 2)); mode = int(rng.integers(0, 3))
    print("seed %d: %s n=%d I=%d O=%d F=%d lut_binarize=%d dx mode %d" % (seed, kind, n, I, O, F, lut_binarize, mode), flush=True)
    idx = synth.wiring(rng, I, O, n); W = synth.lut_tables(rng, O, n)
    ys = stride_fp32(rng, F)
    dy = synth.normal_frames(rng, O, F, ys)
    ops.set_dx_mode(mode)
    rev = ops.reverse_table(dev(idx), I)
    dW = torch.zeros((O, 1 << n), device="cuda")
    if kind in ("st_fp32", "st_bin"):
        binary = kind == "st_bin"
        x = synth.uniform_frames(rng, I, F, ys, -0.1, 1.1)
        y = ops.stochastic_lut_forward(n, dev(x), dev(idx), dev(W), F, binary, bool(lut_binarize))
        y_ref = oracle.stochastic_lut_forward(n, x, idx, W, F, binary, bool(lut_binarize))
        dx = ops.stochastic_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, rev, binary, bool(lut_binarize))
        dx_ref, dW_ref = oracle.stochastic_lut_backward(n, x, dy, idx, W, F, None, binary, bool(lut_binarize))
        assert np.abs(host(y)[:, :F] - y_ref[:, :F]).max() <= 1e-5
        assert rel_err(host(dx)[:, :F], dx_ref[:, :F], float(np.abs(dy).max())) <= 1e-4 and rel_err(host(dW), dW_ref, float(np.abs(dy).max())) <= 1e-4
    elif kind == "st_bit":
        xs = int(rng.choice([synth.frame_stride_bit(F), (F + 31) // 32, (F + 31) // 32 + int(rng.integers(0, 9))]))
        xb = synth.bernoulli_bits(rng, I, F, xs)
        y = ops.bit_stochastic_lut_forward(n, dev(xb), dev(idx), dev(W), F, ys, lut_binarize)
        y_ref = oracle.bit_stochastic_lut_forward(n, xb, idx, W, F, ys, lut_binarize)
        dx = ops.bit_stochastic_lut_backward(n, dev(xb), dev(dy), dev(idx), dev(W), dW, F, rev, lut_binarize)
        dx_ref, dW_ref = oracle.bit_stochastic_lut_backward(n, xb, dy, idx, W, F, None, lut_binarize)
        assert np.abs(host(y)[:, :F] - y_ref[:, :F]).max() <= 1e-5
        assert rel_err(host(dx)[:, :F], dx_ref[:, :F], float(np.abs(dy).max())) <= 1e-4 and rel_err(host(dW), dW_ref, float(np.abs(dy).max())) <= 1e-4
    else:
        if F < 8:
            return
        binary_mode = 1 if kind == "dl_bit" else int(rng.integers(0, 2))
        rm = rng.random(O).astype(np.float32); rv = (rng.random(O) + 0.5).astype(np.float32)
        Wb = (W > 0.5).astype(np.float32) if lut_binarize else W
        # statistics from the oracle first: they say where the batch-norm output t sits; dy is zeroed where t is within
        # rounding of an edge of the hard-tanh window (either side is right there)
        if kind == "dl_fp32":
            x = synth.uniform_frames(rng, I, F, ys, -0.1, 1.1)
            xc = (np.where(x > 0.5, 0.75, 0.25) if binary_mode else np.clip(x, 0, 1))[:, :F]
            _, mean0, rstd0, _, _ = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, 0.3, 0.5, 0.9, 0.25, lut_binarize, binary_mode)
        else:
            xs = synth.frame_stride_bit(F)
            xb = synth.bernoulli_bits(rng, I, F, xs)
            dy = synth.normal_frames(rng, O, F, synth.frame_stride_fp32(F))
            xc = np.where(synth.unpack_bits(xb, F) > 0, 0.75, 0.25)
            _, mean0, rstd0, _, _ = oracle.bit_differentiable_lut_forward_training(n, xb, idx, W, F, rm, rv, lut_binarize=lut_binarize)
        pre = _pre_activation(n, xc, idx, Wb, mean0.astype(np.float64), rstd0.astype(np.float64), 0.3, 0.5)
        edge = (np.abs(pre) < 1e-5) | (np.abs(pre - 1.0) < 1e-5)
        dy[:, :F][edge] = 0.0
        if kind == "dl_fp32":
            y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, 0.3, 0.5, 0.9, 0.25, lut_binarize, binary_mode)
            rmd, rvd = dev(rm), dev(rv)
            y, mean, rstd = ops.differentiable_lut_forward_training(n, dev(x), dev(idx), dev(W), F, rmd, rvd, 0.3, 0.5, 0.9, 0.25, lut_binarize, binary_mode)
            yg, yr = host(y)[:, :F], y_ref[:, :F]
            dx_ref, dW_ref = oracle.differentiable_lut_backward(n, x, dy, idx, W, F, mean_ref, rstd_ref, None, 0.3, 0.5, 0.25, lut_binarize, binary_mode)
            dx = ops.differentiable_lut_backward(n, dev(x), dev(dy), dev(idx), dev(W), dW, F, dev(mean_ref), dev(rstd_ref), rev, 0.3, 0.5, 0.25, lut_binarize, binary_mode)
        else:
            y_ref, mean_ref, rstd_ref, rm_ref, rv_ref = oracle.bit_differentiable_lut_forward_training(n, xb, idx, W, F, rm, rv, lut_binarize=lut_binarize)
            rmd, rvd = dev(rm), dev(rv)
            y, mean, rstd = ops.bit_differentiable_lut_forward_training(n, dev(xb), dev(idx), dev(W), F, rmd, rvd, lut_binarize=lut_binarize)
            yg, yr = synth.unpack_bits(host(y), F), synth.unpack_bits(y_ref, F)
            dx_ref, dW_ref = oracle.bit_differentiable_lut_backward(n, xb, dy, idx, W, F, mean_ref, rstd_ref, lut_binarize=lut_binarize)
            dx = ops.bit_differentiable_lut_backward(n, dev(xb), dev(dy), dev(idx), dev(W), dW, F, dev(mean_ref), dev(rstd_ref), rev, lut_binarize=lut_binarize)
        # the oracle's var = E[y^2] - E[y]^2 (the reference's formula) loses digits when var is small against mean^2
        rtol = 1e-4 + 1e-7 / np.minimum(1.0, 1.0 / rstd_ref.astype(np.float64) ** 2)
        assert rel_err(host(mean), mean_ref) <= 1e-5 and (np.abs(host(rstd) - rstd_ref) <= rtol * rstd_ref).all()
        assert rel_err(host(rmd), rm_ref) <= 1e-5 and rel_err(host(rvd), rv_ref) <= 1e-4
        if binary_mode:
            diff = (yg != yr); near = np.abs(pre - 0.5) < 1e-5
            assert not (diff & ~near).any()
        else:
            tol = 1e-5 * np.maximum(1.0, 0.3 * rstd_ref)[:, None]
            assert (np.abs(yg - yr) <= tol).all()
        if np.abs(dx_ref).max() > 0:
            e1, e2 = rel_err(host(dx)[:, :F], dx_ref[:, :F], float(np.abs(dy).max())), rel_err(host(dW), dW_ref, float(np.abs(dy).max()))
            assert e1 <= 1e-4 and e2 <= 1e-4, (e1, e2)


@pytest.mark.parametrize("block", range(4))
def test_random_shapes(block):
    import torch
    from binarybrain_amd import ops
    try:
        for seed in range(7000 + 40 * block, 7000 + 40 * (block + 1)):
            run_case(ops, torch, seed)
    finally:
        ops.set_dx_mode(0)


def pad(a, stride):
    out = np.zeros((a.shape[0], stride), a.dtype); out[:, :a.shape[1]] = a
    return out


def run_exact_case(ops, seed):
    """the rows whose results are integers, bits or permutations: equal to the oracle bit for bit"""
    F32 = np.float32
    rng = np.random.default_rng(seed)
    kind = str(rng.choice(["binary", "bitbit", "im2col", "col2im", "pool"]))
    if kind == "binary":
        I = int(rng.integers(6, 600)); O = int(rng.integers(1, 400))
        F = int(rng.choice([int(rng.integers(1, 100)), int(rng.integers(100, 3000)), int(rng.integers(3000, 40000))]))
        print("seed %d: binary I=%d O=%d F=%d" % (seed, I, O, F), flush=True)
        words = (F + 31) // 32
        stride = int(rng.choice([synth.frame_stride_bit(F), words, words + int(rng.integers(0, 9))]))
        idx = synth.wiring(rng, I, O); T = synth.truth_tables(rng, O)
        xb = synth.bernoulli_bits(rng, I, F, stride)
        y = ops.binary_lut6_forward(dev(xb), dev(idx), dev(T), F)
        assert np.array_equal(synth.unpack_bits(host(y), F), synth.unpack_bits(oracle.binary_lut6_forward(xb, idx, T, F), F))
    elif kind == "bitbit":
        n = int(rng.integers(2, 7)); I = int(rng.integers(n, 300)); O = int(rng.integers(1, 200)); F = int(rng.integers(1, 6000))
        lb = int(rng.integers(0, 2))
        print("seed %d: bitbit n=%d I=%d O=%d F=%d lb=%d" % (seed, n, I, O, F, lb), flush=True)
        idx = synth.wiring(rng, I, O, n)
        W = synth.lut_tables(rng, O, n)
        xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
        y = ops.bit_bit_stochastic_lut_forward(n, dev(xb), dev(idx), dev(W), F, lb)
        y_ref = oracle.bit_bit_stochastic_lut_forward(n, xb, idx, W, F, lb)
        yf = oracle.bit_stochastic_lut_forward(n, xb, idx, W, F, synth.frame_stride_fp32(F), lb)[:, :F]
        diff = synth.unpack_bits(host(y), F) != synth.unpack_bits(y_ref, F)
        assert not (diff & (np.abs(yf - 0.5) > 1e-6)).any()          # an output bit may differ only where the fp32 output sits on the threshold
    elif kind == "im2col":
        c = int(rng.integers(1, 5)); h = int(rng.integers(1, 20)); w = int(rng.integers(1, 80)); F = int(rng.integers(1, 200))
        fh = int(rng.integers(1, min(h, 4) + 1)); fw = int(rng.integers(1, min(w, 5) + 1))
        ys = int(rng.integers(1, 3)); xs = int(rng.integers(1, 3))
        padm = str(rng.choice(["valid", "same"])); border = str(rng.choice(["reflect_101", "replicate", "constant", "wrap", "reflect"]))
        if padm == "same" and border in ("reflect_101", "reflect") and (h < fh or w < fw or h < 2 or w < 2):
            return
        print("seed %d: im2col c=%d h=%d w=%d F=%d f=%dx%d s=%d,%d %s %s" % (seed, c, h, w, F, fh, fw, ys, xs, padm, border), flush=True)
        x = rng.random((c * h * w, F)).astype(F32)
        y_ref = oracle.im2col_forward(x, c, h, w, F, fh, fw, ys, xs, padm, border, 0.25)
        of = y_ref.shape[1]
        y = host(ops.im2col_forward(dev(pad(x, synth.frame_stride_fp32(F))), c, h, w, F, fh, fw, ys, xs, padm, border, 0.25))
        assert np.array_equal(y[:, :of], y_ref)
        dy = rng.standard_normal((c * fh * fw, of)).astype(F32)
        dx_ref = oracle.im2col_backward(dy, c, h, w, F, fh, fw, ys, xs, padm)
        dx = host(ops.im2col_backward(dev(pad(dy, synth.frame_stride_fp32(of))), c, h, w, F, fh, fw, ys, xs, padm))
        assert np.array_equal(dx[:, :F], dx_ref)
        xb = synth.bernoulli_bits(rng, c * h * w, F, synth.frame_stride_bit(F))
        yb_ref = oracle.im2col_forward(xb, c, h, w, F, fh, fw, ys, xs, padm, border, bit=True)
        yb = host(ops.im2col_forward(dev(xb), c, h, w, F, fh, fw, ys, xs, padm, border))
        assert np.array_equal(synth.unpack_bits(yb, of), synth.unpack_bits(yb_ref, of))
    elif kind == "col2im":
        c = int(rng.integers(1, 40)); h = int(rng.integers(1, 20)); w = int(rng.integers(1, 20)); F = int(rng.integers(1, 40))
        print("seed %d: col2im c=%d h=%d w=%d F=%d" % (seed, c, h, w, F), flush=True)
        x = rng.random((c, F * h * w)).astype(F32)
        y_ref = oracle.col2im_forward(x, c, h, w, F)
        y = host(ops.col2im_forward(dev(pad(x, synth.frame_stride_fp32(F * h * w))), c, h, w, F))
        assert np.array_equal(y[:, :F], y_ref[:, :F])
        dy = rng.standard_normal((c * h * w, F)).astype(F32)
        dx_ref = oracle.col2im_backward(dy, c, h, w, F)
        dx = host(ops.col2im_backward(dev(pad(dy, synth.frame_stride_fp32(F))), c, h, w, F))
        assert np.array_equal(dx[:, :F * h * w], dx_ref[:, :F * h * w])
    else:
        c = int(rng.integers(1, 20)); h = int(rng.integers(1, 24)); w = int(rng.integers(1, 24)); F = int(rng.integers(1, 300))
        print("seed %d: pool c=%d h=%d w=%d F=%d" % (seed, c, h, w, F), flush=True)
        x = rng.random((c * h * w, F)).astype(F32)
        y_ref = oracle.stochastic_maxpool2x2_forward(x, c, h, w, F)
        xd = dev(pad(x, synth.frame_stride_fp32(F)))
        y = host(ops.stochastic_maxpool2x2_forward(xd, c, h, w, F))
        assert np.array_equal(y[:, :F], y_ref[:, :F])
        dy = rng.standard_normal((y_ref.shape[0], F)).astype(F32)
        dx_ref = oracle.stochastic_maxpool2x2_backward(x, dy, c, h, w, F)
        dx = host(ops.stochastic_maxpool2x2_backward(xd, dev(pad(dy, synth.frame_stride_fp32(F))), c, h, w, F))
        assert np.array_equal(dx[:, :F], dx_ref[:, :F])

def test_random_shapes_of_the_exact_rows():
    from binarybrain_amd import ops
    for seed in range(9000, 9400):
        run_exact_case(ops, seed)


def run_tail_case(ops, torch, seed):
    """AverageLut, MaxLut and accuracy bit-exact, the loss at the tolerances of tests/test_gpu_tail.py, the normalisation at those of
    tests/test_gpu_stochastic_bn.py, Adam bit-exact"""
    import test_gpu_tail as tail
    F32 = np.float32
    rng = np.random.default_rng(seed)
    kind = str(rng.choice(["average", "loss", "adam"]))
    if seed >= 11150:           # the first 150 seeds keep the cases they always drew; later ones also draw the two newer kinds
        kind = str(rng.choice([kind, "maxlut", "bn"], p=[0.4, 0.3, 0.3]))
    if kind == "maxlut":
        n = int(rng.choice([int(rng.integers(1, 17)), int(rng.integers(17, 200))])); I = int(rng.integers(1, 400)); O = int(rng.integers(1, 120))
        F = int(rng.integers(1, 1500))
        print("seed %d: maxlut n=%d I=%d O=%d F=%d" % (seed, n, I, O, F), flush=True)
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        stride = synth.frame_stride_fp32(F)
        x = (rng.random((I, F)) * 3 - 2).astype(F32)
        x[rng.random(x.shape) < 0.1] = 0.0
        x[:, ::3] = np.round(x[:, ::3])
        x = tail._pad(x, stride)
        dy = tail._pad(rng.standard_normal((O, F)).astype(F32), stride)
        for bin_in in (False, True):
            for bin_out in (False, True):
                y = host(ops.max_lut_forward(dev(x), dev(idx), F, bin_in, bin_out))
                assert np.array_equal(y[:, :F], oracle.max_lut_forward(x, idx, F, bin_in, bin_out)[:, :F]), (bin_in, bin_out)
            dx = host(ops.max_lut_backward(dev(x), dev(dy), dev(idx), F, bin_in))
            assert np.array_equal(dx, oracle.max_lut_backward(x, dy, idx, F, bin_in)), bin_in
        xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F), p=float(rng.choice([0.05, 0.3, 0.9])))
        yb = host(ops.bit_max_lut_forward(dev(xb), dev(idx), F))
        assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(oracle.bit_max_lut_forward(xb, idx, F), F))
        assert np.array_equal(host(ops.bit_max_lut_backward(dev(xb), dev(dy), dev(idx), F)), oracle.bit_max_lut_backward(xb, dy, idx, F))
    elif kind == "bn":
        import test_gpu_stochastic_bn as bn
        nodes = int(rng.integers(1, 300)); F = int(rng.choice([int(rng.integers(2, 70)), int(rng.integers(64, 3000)), int(rng.integers(3000, 20000))]))
        stride = int(rng.choice([synth.frame_stride_fp32(F), F, F + int(rng.integers(1, 9))]))
        gamma = float(rng.choice([0.2, 0.3, 1.0])); beta = float(rng.choice([0.5, 0.0])); momentum = float(rng.choice([0.9, 0.0, 0.99]))
        print("seed %d: bn nodes=%d F=%d stride=%d gamma=%g beta=%g momentum=%g" % (seed, nodes, F, stride, gamma, beta, momentum), flush=True)
        x = bn._pad((rng.random((nodes, F)) * float(rng.choice([1.0, 0.05]))).astype(F32), stride)
        dy = bn._pad(rng.standard_normal((nodes, F)).astype(F32), stride)
        rm0 = rng.standard_normal(nodes).astype(F32); rv0 = (rng.random(nodes) + 0.5).astype(F32)
        want = oracle.stochastic_bn_forward_training(x, rm0, rv0, gamma, beta, momentum, F)
        rm = dev(rm0); rv = dev(rv0)
        y, mean, rstd = ops.stochastic_bn_forward_training(dev(x), rm, rv, F, gamma, beta, momentum)
        bn.check_forward(host(y), host(mean), host(rstd), host(rm), host(rv), want, x, gamma, F)
        dx = host(ops.stochastic_bn_backward(dev(x), dev(dy), dev(want[1]), dev(want[2]), F, gamma))
        bn.check_backward(dx, oracle.stochastic_bn_backward(x, dy, want[1], want[2], gamma, F), dy, want[2], gamma, x, F)
        yi = host(ops.stochastic_bn_forward_inference(dev(x), dev(rm0), dev(rv0), F, gamma, beta))
        wi = oracle.stochastic_bn_forward_inference(x, rm0, rv0, gamma, beta, F)
        assert np.all(np.abs(yi[:, :F] - wi[:, :F]) <= 2e-6 * (np.abs(wi[:, :F]) + 1.0))
    elif kind == "average":
        n = int(rng.choice([int(rng.integers(1, 17)), int(rng.integers(17, 400))])); I = int(rng.integers(1, 400)); O = int(rng.integers(1, 120))
        F = int(rng.integers(1, 1500))
        print("seed %d: average n=%d I=%d O=%d F=%d" % (seed, n, I, O, F), flush=True)
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        stride = synth.frame_stride_fp32(F)
        x = tail._pad((rng.random((I, F)) * 2 - 1).astype(F32), stride)
        x[rng.random(x.shape) < 0.05] = 0.0
        dy = tail._pad(rng.standard_normal((O, F)).astype(F32), stride)
        for bin_in in (False, True):
            for bin_out in (False, True):
                mean = bool((bin_in + 2 * bin_out + F) & 1)          # both conventions for the un-binarized output
                y = host(ops.average_lut_forward(dev(x), dev(idx), F, bin_in, bin_out, mean=mean))
                assert np.array_equal(y[:, :F], oracle.average_lut_forward(x, idx, F, bin_in, bin_out, mean=mean)[:, :F]), (bin_in, bin_out, mean)
        dx = host(ops.average_lut_backward(dev(dy), dev(idx), I, F))
        assert np.array_equal(dx, oracle.average_lut_backward(dy, idx, I, F))
        xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
        yb = host(ops.bit_average_lut_forward(dev(xb), dev(idx), F))
        assert np.array_equal(synth.unpack_bits(yb, F), synth.unpack_bits(oracle.bit_average_lut_forward(xb, idx, F), F))
    elif kind == "loss":
        ch = int(rng.choice([int(rng.integers(1, 12)), int(rng.integers(12, 300))])); pix = int(rng.choice([1, int(rng.integers(1, 40))]))
        F = int(rng.integers(1, 600))
        sharp = bool(rng.integers(0, 2)); weighted = bool(rng.integers(0, 2))
        print("seed %d: loss ch=%d pix=%d F=%d sharp=%d weighted=%d" % (seed, ch, pix, F, sharp, weighted), flush=True)
        y = (rng.standard_normal((ch * pix, F)) * (30.0 if sharp else 1.0)).astype(F32)
        t = tail._targets(rng, ch, pix, F, weighted=weighted)
        if not t.any():
            t[0, 0] = 1
        tail._check_loss(ops, y, t, ch, pix, F, synth.frame_stride_fp32(F))
    else:
        k = int(rng.integers(1, 6))
        shapes = [(int(rng.integers(1, 3000)),) if rng.integers(0, 2) else (int(rng.integers(1, 300)), 64) for _ in range(k)]
        lr = float(rng.choice([0.001, 0.01, 0.1])); b1 = float(rng.choice([0.9, 0.5])); b2 = float(rng.choice([0.999, 0.9]))
        steps = int(rng.integers(1, 5))
        print("seed %d: adam %s lr=%g b=%g,%g steps=%d" % (seed, shapes, lr, b1, b2, steps), flush=True)
        p0 = [rng.random(s).astype(F32) for s in shapes]
        params = [dev(a.copy()) for a in p0]
        grads = [torch.zeros_like(p) for p in params]
        st = ops.AdamState(params, grads, lr, b1, b2)
        gs = [[(rng.standard_normal(s) * 0.1).astype(F32) for s in shapes] for _ in range(steps)]
        for step in gs:
            for g, a in zip(grads, step):
                g.copy_(dev(a))
            st.step()
        for i, s in enumerate(shapes):
            ref, m, v = oracle.adam_steps(p0[i].ravel(), [step[i].ravel() for step in gs], lr, b1, b2)
            assert np.array_equal(host(params[i]).ravel(), ref), s
            assert np.array_equal(host(st.m[i]).ravel(), m) and np.array_equal(host(st.v[i]).ravel(), v)

def test_random_shapes_of_the_classifier_tail_and_adam():
    import torch
    from binarybrain_amd import ops
    for seed in range(11000, 11300):
        run_tail_case(ops, torch, seed)


def run_plumbing_case(ops, seed):
    """RealToBinary, BinaryToReal, Binarize / HardTanh, MaxPooling and UpSampling at random shapes, row pitches and parameters: all of them
    bit for bit against the oracle"""
    F32 = np.float32
    rng = np.random.default_rng(seed)
    kind = str(rng.choice(["real_to_binary", "binary_to_real", "activation", "max_pooling", "up_sampling"]))

    def pitch(n):
        return int(rng.choice([synth.frame_stride_fp32(n), n, n + int(rng.integers(1, 9))]))

    def words(n):
        return int(rng.choice([synth.frame_stride_bit(n), (n + 31) // 32, (n + 31) // 32 + int(rng.integers(1, 4))]))

    if kind == "real_to_binary":
        d = int(rng.integers(1, 5)); p = int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(40, 900))])); F = int(rng.integers(1, 300))
        fm = int(rng.choice([1, 2, 7, 15, int(rng.integers(1, 70))])); dm = int(rng.choice([1, 1, 2, int(rng.integers(1, 6))]))
        lo, hi = [(0.0, 1.0), (-1.0, 1.0), (0.0, 255.0), (0.1, 0.9)][int(rng.integers(0, 4))]
        binarize = bool(rng.integers(0, 2))
        print("seed %d: real_to_binary d=%d p=%d F=%d fm=%d dm=%d range=(%g, %g) binarize=%d" % (seed, d, p, F, fm, dm, lo, hi, binarize), flush=True)
        x = pad((rng.random((d * p, F)) * (hi - lo) * 1.2 + lo - 0.1 * (hi - lo)).astype(F32), pitch(F))
        ys, ws = pitch(F * fm), words(F * fm)
        got = host(ops.real_to_binary_forward(dev(x), d, p, F, fm, dm, lo, hi, binarize=binarize, y_stride=ys))
        assert np.array_equal(got[:, :F * fm], oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=binarize, y_stride=ys)[:, :F * fm])
        got = host(ops.real_to_binary_forward(dev(x), d, p, F, fm, dm, lo, hi, binarize=binarize, bit=True, y_stride=ws))
        assert np.array_equal(got, oracle.real_to_binary_forward(x, d, p, F, fm, dm, lo, hi, binarize=binarize, bit=True, y_stride=ws))
    elif kind == "binary_to_real":
        O = int(rng.integers(1, 200)); mux = int(rng.choice([1, 1, 7, int(rng.integers(1, 12))])); Fy = int(rng.integers(1, 300))
        fm = int(rng.choice([1, 2, 7, 15, 32, int(rng.integers(1, 70))]))
        I, F = O * mux, Fy * fm
        print("seed %d: binary_to_real I=%d O=%d Fy=%d fm=%d" % (seed, I, O, Fy, fm), flush=True)
        xs, ys, ws = pitch(F), pitch(Fy), words(F)
        x = pad(rng.standard_normal((I, F)).astype(F32), xs)
        x[:, F:] = 3.0
        x[rng.random(x.shape) < 0.1] = 0.0
        assert np.array_equal(host(ops.binary_to_real_forward(dev(x), O, Fy, fm, y_stride=ys))[:, :Fy], oracle.binary_to_real_forward(x, O, Fy, fm, y_stride=ys)[:, :Fy])
        xb = synth.bernoulli_bits(rng, I, F, ws, p=float(rng.choice([0.1, 0.5, 0.9])))
        xb[:, (F + 31) // 32:] = -1
        assert np.array_equal(host(ops.binary_to_real_forward(dev(xb), O, Fy, fm, y_stride=ys))[:, :Fy],
                              oracle.binary_to_real_forward(xb, O, Fy, fm, bit=True, y_stride=ys)[:, :Fy])
        dy = pad(rng.standard_normal((O, Fy)).astype(F32), ys)
        assert np.array_equal(host(ops.binary_to_real_backward(dev(dy), I, Fy, fm, x_stride=xs))[:, :F], oracle.binary_to_real_backward(dy, I, Fy, fm, x_stride=xs)[:, :F])
    elif kind == "activation":
        nodes = int(rng.integers(1, 400)); F = int(rng.choice([int(rng.integers(1, 70)), int(rng.integers(64, 5000))]))
        lo, hi = sorted(float(v) for v in rng.standard_normal(2)); th = float(rng.standard_normal() * 0.3)
        if lo == hi:
            hi = lo + 1.0
        print("seed %d: activation nodes=%d F=%d window=(%g, %g) th=%g" % (seed, nodes, F, lo, hi, th), flush=True)
        st = pitch(F)
        x = pad(rng.standard_normal((nodes, F)).astype(F32), st); dy = pad(rng.standard_normal((nodes, F)).astype(F32), st)
        x.flat[:4] = [lo, hi, th, np.nan]
        assert np.array_equal(host(ops.binarize_forward(dev(x), F, th, -1.0, 1.0))[:, :F], oracle.binarize_forward(x, F, th, -1.0, 1.0)[:, :F])
        ws = words(F)
        assert np.array_equal(host(ops.binarize_forward(dev(x), F, th, bit=True, y_stride=ws)), oracle.binarize_forward(x, F, th, bit=True, y_stride=ws))
        assert np.array_equal(host(ops.hard_tanh_forward(dev(x), F, lo, hi))[:, :F], oracle.hard_tanh_forward(x, F, lo, hi)[:, :F], equal_nan=True)
        assert np.array_equal(host(ops.hard_tanh_backward(dev(x), dev(dy), F, lo, hi))[:, :F], oracle.hard_tanh_backward(x, dy, F, lo, hi)[:, :F])
    elif kind == "max_pooling":
        c = int(rng.integers(1, 12)); h = int(rng.integers(1, 20)); w = int(rng.integers(1, 20)); fh = int(rng.choice([1, 2, 2, 3, int(rng.integers(1, 6))]))
        fw = int(rng.choice([1, 2, 2, 3, int(rng.integers(1, 6))])); F = int(rng.integers(1, 400))
        print("seed %d: max_pooling c=%d h=%d w=%d filter=%dx%d F=%d" % (seed, c, h, w, fh, fw, F), flush=True)
        st = pitch(F)
        x = pad(rng.standard_normal((c * h * w, F)).astype(F32), st)
        x[rng.random(x.shape) < 0.2] = 0.5
        O = c * ((h + fh - 1) // fh) * ((w + fw - 1) // fw)
        dy = pad(rng.standard_normal((O, F)).astype(F32), st)
        y, arg = ops.max_pooling_forward(dev(x), c, h, w, fh, fw, F)
        y_ref, arg_ref = oracle.max_pooling_forward(x, c, h, w, fh, fw, F)
        assert np.array_equal(host(y)[:, :F], y_ref[:, :F]) and np.array_equal(host(arg)[:, :F], arg_ref[:, :F])
        assert np.array_equal(host(ops.max_pooling_backward(arg, dev(dy), c, h, w, fh, fw, F))[:, :F], oracle.max_pooling_backward(arg_ref, dy, c, h, w, fh, fw, F)[:, :F])
        xb = synth.bernoulli_bits(rng, c * h * w, F, words(F), p=float(rng.choice([0.05, 0.3, 0.8])))
        nw = (F + 31) // 32
        assert np.array_equal(host(ops.bit_max_pooling_forward(dev(xb), c, h, w, fh, fw, F))[:, :nw], oracle.bit_max_pooling_forward(xb, c, h, w, fh, fw, F)[:, :nw])
        assert np.array_equal(host(ops.bit_max_pooling_backward(dev(xb), dev(dy), c, h, w, fh, fw, F))[:, :F],
                              oracle.bit_max_pooling_backward(xb, dy, c, h, w, fh, fw, F)[:, :F])
    else:
        c = int(rng.integers(1, 12)); h = int(rng.integers(1, 12)); w = int(rng.integers(1, 12)); fh = int(rng.integers(1, 5)); fw = int(rng.integers(1, 5))
        F = int(rng.integers(1, 400)); fill = bool(rng.integers(0, 2))
        print("seed %d: up_sampling c=%d h=%d w=%d filter=%dx%d F=%d fill=%d" % (seed, c, h, w, fh, fw, F, fill), flush=True)
        st = pitch(F)
        x = pad(rng.standard_normal((c * h * w, F)).astype(F32), st)
        dy = pad(rng.standard_normal((c * h * fh * w * fw, F)).astype(F32), st)
        assert np.array_equal(host(ops.up_sampling_forward(dev(x), c, h, w, fh, fw, F, fill))[:, :F], oracle.up_sampling_forward(x, c, h, w, fh, fw, F, fill)[:, :F])
        assert np.array_equal(host(ops.up_sampling_backward(dev(dy), c, h, w, fh, fw, F, fill))[:, :F], oracle.up_sampling_backward(dy, c, h, w, fh, fw, F, fill)[:, :F])
        xb = synth.bernoulli_bits(rng, c * h * w, F, words(F))
        nw = (F + 31) // 32
        assert np.array_equal(host(ops.up_sampling_forward(dev(xb), c, h, w, fh, fw, F, fill))[:, :nw], oracle.up_sampling_forward(xb, c, h, w, fh, fw, F, fill, bit=True)[:, :nw])


def test_random_shapes_of_the_converters_activations_and_pooling():
    from binarybrain_amd import ops
    for seed in range(13000, 13250):
        run_plumbing_case(ops, seed)


def run_shuffle_case(ops, seed):
    """Shuffle at random node counts, units and row pitches, fp32 rows and packed rows: whole rows bit for bit against the oracle"""
    rng = np.random.default_rng(seed)
    unit = int(rng.choice([1, 2, 3, 7, 32, int(rng.integers(1, 100))])); group = int(rng.choice([1, 2, 5, 36, int(rng.integers(1, 200))]))
    nodes = unit * group
    F = int(rng.integers(1, 600))
    stride = int(rng.choice([synth.frame_stride_fp32(F), F, F + int(rng.integers(1, 9))]))
    print("seed %d: shuffle nodes=%d unit=%d F=%d stride=%d" % (seed, nodes, unit, F, stride), flush=True)
    x = rng.integers(-2**31, 2**31, (nodes, stride)).astype(np.int32)
    assert np.array_equal(host(ops.shuffle_forward(dev(x), unit, F)), oracle.shuffle_forward(x, unit))
    assert np.array_equal(host(ops.shuffle_backward(dev(x), unit, F)), oracle.shuffle_backward(x, unit))
    xf = x.view(np.float32)                                              # the same words as fp32 rows (NaN patterns included)
    assert np.array_equal(host(ops.shuffle_forward(dev(xf), unit, F)).view(np.int32), oracle.shuffle_forward(x, unit))


def test_random_shapes_of_shuffle():
    from binarybrain_amd import ops
    for seed in range(14000, 14100):
        run_shuffle_case(ops, seed)


def test_extended_random_run():
    """The same five generators over further seeds, for a longer run on the device: set BBHIP_EXTENDED_CASES=N (N cases of each
    generator, at most 200 000; seeds continue after the ones above).  Stops at the first failing case, whose seed the case
    prints.  Without the variable the test is skipped, so the default suite stays short:
        BBHIP_EXTENDED_CASES=10000 python -u -m pytest tests/test_gpu_random_shapes.py -k extended -x -s"""
    import os
    count = int(os.environ.get("BBHIP_EXTENDED_CASES", "0") or 0)
    if count <= 0:
        pytest.skip("BBHIP_EXTENDED_CASES is not set")
    count = min(count, 200000)
    import torch
    from binarybrain_amd import ops
    try:
        for k in range(count):
            run_case(ops, torch, 100000 + k)
            run_exact_case(ops, 400000 + k)
            run_tail_case(ops, torch, 700000 + k)
            run_plumbing_case(ops, 900000 + k)
            run_shuffle_case(ops, 1200000 + k)
            if (k + 1) % 500 == 0:
                print("extended run: %d of %d" % (k + 1, count), flush=True)
    finally:
        ops.set_dx_mode(0)
    print("extended run: %d cases of each generator, no mismatch" % count)
