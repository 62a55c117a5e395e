"""The binarized output of a forward call written as packed bits as well (bbhip_HintPackedOutput), handed to the next layer as the packed
copy of its input (bbhip_HintPackedInput with holds_input = 1): no result changes by a bit, the packed copy equals the bits of y > 0.5,
and the next layer's forward and backward calls read it instead of packing.  Also: the table gradient written instead of accumulated
(bbhip_HintTableGradientOverwrite) equals zero-fill + accumulate."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


# (one unit per node with the statistics summed by the output wavefront; several units per node; ragged last words; narrow layers)
@pytest.mark.parametrize("shape", [(64, 48, 1024), (27, 216, 5000), (784, 300, 200), (100, 70, 37), (50, 9, 2048 + 33)])
@pytest.mark.parametrize("kind", ["training", "inference", "no_bn"])
def test_two_layers_with_and_without_the_packed_output(ops, shape, kind):
    import torch
    I, O, F = shape
    O2 = 40
    rng = np.random.default_rng(I * 3 + O + F)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S))
    dy = dev(synth.normal_frames(rng, O2, F, S))
    idx1, idx2 = dev(synth.wiring(rng, I, O)), dev(synth.wiring(rng, O, O2))
    W1 = dev((0.5 + 0.2 * rng.standard_normal((O, 64))).astype(np.float32))
    W2 = dev((0.5 + 0.2 * rng.standard_normal((O2, 64))).astype(np.float32))
    rev1, rev2 = ops.reverse_table(idx1, I), ops.reverse_table(idx2, O)
    ops.set_dx_mode(0)

    def forward(xx, idx, W, rm, rv, **kw):
        if kind == "training":
            return ops.differentiable_lut_forward_training(6, xx, idx, W, F, rm, rv, **kw)
        if kind == "inference":
            return ops.differentiable_lut_forward_inference(6, xx, idx, W, F, rm, rv, **kw), None, None
        return ops.differentiable_lut_forward_nobn(6, xx, idx, W, F, **kw), None, None

    def run(with_bits):
        rm1 = torch.full((O,), 0.5, device="cuda"); rv1 = torch.full((O,), 0.01, device="cuda")
        rm2 = torch.full((O2,), 0.5, device="cuda"); rv2 = torch.full((O2,), 0.01, device="cuda")
        out = []
        p0 = ops.packed_input_buffer(I, F) if with_bits else None
        p1 = ops.packed_input_buffer(O, F) if with_bits else None
        if with_bits:
            p1.fill_(0x5a5a5a5a)
        y1, m1, r1 = forward(x, idx1, W1, rm1, rv1, packed=p0, packed_out=p1)
        y2, m2, r2 = forward(y1, idx2, W2, rm2, rv2, packed=p1, packed_holds=with_bits)
        out += [y1[:, :F], y2[:, :F], rm1, rv1, rm2, rv2]
        if kind == "training":
            dW2 = torch.zeros((O2, 64), device="cuda"); dW1 = torch.zeros((O, 64), device="cuda")
            dx2 = ops.differentiable_lut_backward(6, y1, dy, idx2, W2, dW2, F, m2, r2, rev2, packed=p1)
            dx1 = ops.differentiable_lut_backward(6, x, dx2, idx1, W1, dW1, F, m1, r1, rev1, packed=p0)
            out += [m1, r1, m2, r2, dx2[:, :F], dx1[:, :F], dW1, dW2]
        return [host(t) for t in out], p1, y1

    plain, _, _ = run(False)
    kept, p1, y1 = run(True)
    for k, (a, b) in enumerate(zip(plain, kept)):
        assert np.array_equal(a, b), k
    # the packed copy: the bits of y1 > 0.5 in whole rows, nothing but zeros behind the last frame
    want = oracle.binarize_forward(host(y1), F, 0.5, bit=True)
    nw = (F + 31) // 32
    got = host(p1)
    assert np.array_equal(got[:, :nw], want[:, :nw])
    assert not got[:, nw:].any()


def test_the_packed_copy_is_what_the_next_layer_reads(ops):
    """with another layer's bits in the buffer that is declared to hold the input, the output changes: the call did not pack x again"""
    import torch
    I, O, F = 60, 50, 512
    rng = np.random.default_rng(5)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S)); idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O))
    y0 = ops.differentiable_lut_forward_nobn(6, x, idx, W, F)
    bits = ops.packed_input_buffer(I, F)
    y1 = ops.differentiable_lut_forward_nobn(6, x, idx, W, F, packed=bits)                       # fills it
    y2 = ops.differentiable_lut_forward_nobn(6, x, idx, W, F, packed=bits, packed_holds=True)    # reads it
    assert torch.equal(y0[:, :F], y1[:, :F]) and torch.equal(y0[:, :F], y2[:, :F])      # (what lies past the last frame of a row is not specified)
    bits ^= 0x0f0f0f0f
    y3 = ops.differentiable_lut_forward_nobn(6, x, idx, W, F, packed=bits, packed_holds=True)
    assert not torch.equal(y0[:, :F], y3[:, :F])
    # a buffer that does not fit the call (another row count) is neither read nor written
    odd = torch.full((O + 1, bits.shape[1]), 0x33333333, dtype=torch.int32, device="cuda")
    from binarybrain_amd.capi import lib
    from binarybrain_amd.ops import ptr
    lib().bbhip_HintPackedOutput(ptr(odd), O + 1, odd.shape[1])
    y4 = ops.differentiable_lut_forward_nobn(6, x, idx, W, F)
    assert torch.equal(y0[:, :F], y4[:, :F]) and int((odd != 0x33333333).sum()) == 0


@pytest.mark.parametrize("batch_norm", [True, False])
@pytest.mark.parametrize("dx_mode", [0, 1, 2])
def test_table_gradient_written_instead_of_accumulated(ops, batch_norm, dx_mode):
    import torch
    I, O, F = 70, 90, 700
    rng = np.random.default_rng(11 + dx_mode)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S)); dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O)); rev = ops.reverse_table(idx, I)
    ops.set_dx_mode(dx_mode)
    try:
        def run(dW, overwrite):
            if batch_norm:
                rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
                _, mean, rstd = ops.differentiable_lut_forward_training(6, x, idx, W, F, rm, rv, binary_mode=False)
                return ops.differentiable_lut_backward(6, x, dy, idx, W, dW, F, mean, rstd, rev, binary_mode=False, overwrite_dw=overwrite)
            return ops.stochastic_lut_backward(6, x, dy, idx, W, dW, F, rev, overwrite_dw=overwrite)
        dW0 = torch.zeros((O, 64), device="cuda")
        dx0 = run(dW0, False)
        dW1 = torch.full((O, 64), 123.0, device="cuda")
        dx1 = run(dW1, True)
        if dx_mode == 1:        # atomics: not reproducible bit for bit between two runs
            assert float((dW0 - dW1).abs().max()) <= 1e-5 * float(dW0.abs().max())
        else:
            assert torch.equal(dW0, dW1) and torch.equal(dx0[:, :F], dx1[:, :F])
        # and the hint is spent: the next call accumulates again
        dx2 = run(dW1, False)
        assert float((dW1 - 2 * dW0).abs().max()) <= 1e-5 * float(dW0.abs().max())
    finally:
        ops.set_dx_mode(0)
