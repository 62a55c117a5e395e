"""One parity case on two-valued inputs (packed bits, and fp32 frames in binary mode), forward and backward, StochasticLut and
DifferentiableLut, plus continuous fp32 frames and BinaryLut6, against the CPU oracle.  Run as a script by test_gpu_tunables.py in a process of its own, because the
library reads its environment switches once: with BBHIP_CORNER=2 BBHIP_PACK=2 the polynomial kernels serve these inputs."""
import sys

import numpy as np

import oracle
from binarybrain_amd import ops, synth
from util import assert_bwd, assert_fwd, dev, host


def main():
    import torch
    ops.set_dx_mode(0)
    rng = np.random.default_rng(12)
    I, O, F = 48, 40, 1300
    idx = synth.wiring(rng, I, O, 6); W = synth.lut_tables(rng, O, 6)
    ys = synth.frame_stride_fp32(F)
    dy = synth.normal_frames(rng, O, F, ys)
    rev = ops.reverse_table(dev(idx), I)

    # packed bits, StochasticLut
    xb = synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))
    y = ops.bit_stochastic_lut_forward(6, dev(xb), dev(idx), dev(W), F, ys, 0)
    assert_fwd(host(y)[:, :F], oracle.bit_stochastic_lut_forward(6, xb, idx, W, F, ys, 0)[:, :F], "bit")
    dx_ref, dW_ref = oracle.bit_stochastic_lut_backward(6, xb, dy, idx, W, F, None, 0)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.bit_stochastic_lut_backward(6, dev(xb), dev(dy), dev(idx), dev(W), dW, F, rev, 0)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "bit dx"); assert_bwd(host(dW), dW_ref, "bit dW")

    # fp32 frames in binary mode, DifferentiableLut with batch-norm
    x = synth.uniform_frames(rng, I, F, ys)
    z, o = np.zeros(O, np.float32), np.ones(O, np.float32)
    y_ref, m_ref, r_ref, _, _ = oracle.differentiable_lut_forward_training(6, x, idx, W, F, z, o)
    y, mean, rstd = ops.differentiable_lut_forward_training(6, dev(x), dev(idx), dev(W), F, torch.zeros(O, device="cuda"), torch.ones(O, device="cuda"))
    assert np.mean(host(y)[:, :F] != y_ref[:, :F]) < 1e-3
    assert np.allclose(host(mean), m_ref, rtol=1e-4, atol=1e-6) and np.allclose(host(rstd), r_ref, rtol=1e-4)
    dx_ref, dW_ref = oracle.differentiable_lut_backward(6, x, dy, idx, W, F, m_ref, r_ref)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.differentiable_lut_backward(6, dev(x), dev(dy), dev(idx), dev(W), dW, F, dev(m_ref), dev(r_ref), rev)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "binary dx"); assert_bwd(host(dW), dW_ref, "binary dW")
    # the binarized output as packed bits as well, under whichever kernels serve the call: the bits of y > 0.5, zeros behind the last frame
    for kw in ({}, {"packed": ops.packed_input_buffer(I, F)}):
        bits = ops.packed_input_buffer(O, F); bits.fill_(0x5a5a5a5a)
        y2, _, _ = ops.differentiable_lut_forward_training(6, dev(x), dev(idx), dev(W), F, torch.zeros(O, device="cuda"), torch.ones(O, device="cuda"),
                                                           packed_out=bits, **kw)
        assert torch.equal(y2[:, :F], y[:, :F])
        nw = (F + 31) // 32
        assert np.array_equal(host(bits)[:, :nw], oracle.binarize_forward(host(y2), F, 0.5, bit=True)[:, :nw]) and not host(bits)[:, nw:].any()
    # continuous fp32 frames (the polynomial kernels under whatever unit sizes the environment sets)
    xc = synth.uniform_frames(rng, I, F, ys, -0.1, 1.1)
    assert_fwd(host(ops.stochastic_lut_forward(6, dev(xc), dev(idx), dev(W), F))[:, :F], oracle.stochastic_lut_forward(6, xc, idx, W, F, 0, 0, 0.25, False)[:, :F], "fp32")
    dx_ref, dW_ref = oracle.stochastic_lut_backward(6, xc, dy, idx, W, F, None, 0, 0, 0.25, False)
    dW = dev(np.zeros((O, 64), np.float32))
    dx = ops.stochastic_lut_backward(6, dev(xc), dev(dy), dev(idx), dev(W), dW, F, rev)
    assert_bwd(host(dx)[:, :F], dx_ref[:, :F], "fp32 dx"); assert_bwd(host(dW), dW_ref, "fp32 dW")

    # BinaryLut6
    T = rng.integers(-2**31, 2**31, (O, 2)).astype(np.int32)
    Fb = 70000
    xbb = synth.bernoulli_bits(rng, I, Fb, synth.frame_stride_bit(Fb))
    yb = ops.binary_lut6_forward(dev(xbb), dev(idx), dev(T), Fb)
    assert np.array_equal(host(yb), oracle.binary_lut6_forward(xbb, idx, T, Fb))
    from binarybrain_amd import capi
    print("switches corner=%d pack=%d" % (capi.lib().bbhip_GetSwitch(b"corner"), capi.lib().bbhip_GetSwitch(b"pack")))
    print("two-valued case ok")


if __name__ == "__main__":
    sys.exit(main())
