"""The caller-owned packed copy of a binarized fp32 input (bbhip_HintPackedInput): the forward call fills the caller's buffer with the
bits of x > 0.5, the backward call reads them instead of packing x again, and neither changes a bit of any result; a buffer that does
not fit the call is ignored."""
import numpy as np
import pytest

import oracle
from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


@pytest.mark.parametrize("shape", [(64, 48, 1024), (27, 216, 5000), (784, 300, 200), (100, 70, 37)])
@pytest.mark.parametrize("batch_norm", [True, False])
def test_results_do_not_depend_on_the_packed_copy(ops, shape, batch_norm):
    import torch
    I, O, F = shape
    rng = np.random.default_rng(I + O + F)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S))
    dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O))
    W = dev(synth.lut_tables(rng, O))
    rev = ops.reverse_table(idx, I)
    ops.set_dx_mode(0)

    def frames(t):
        a = host(t)
        return a[:, :F] if a.ndim == 2 and a.shape[1] == S else a       # what lies past the last frame of a row is not specified

    def run(packed_fwd, packed_bwd):
        dW = torch.zeros((O, 64), device="cuda")
        if batch_norm:
            rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
            y, mean, rstd = ops.differentiable_lut_forward_training(6, x, idx, W, F, rm, rv, packed=packed_fwd)
            dx = ops.differentiable_lut_backward(6, x, dy, idx, W, dW, F, mean, rstd, rev, packed=packed_bwd)
            return [frames(t) for t in (y, mean, rstd, rm, rv, dx, dW)]
        y = ops.stochastic_lut_forward(6, x, idx, W, F, input_binary=True, packed=packed_fwd)
        dx = ops.stochastic_lut_backward(6, x, dy, idx, W, dW, F, rev, input_binary=True, packed=packed_bwd)
        return [frames(t) for t in (y, dx, dW)]

    plain = run(None, None)
    packed = ops.packed_input_buffer(I, F)
    packed.fill_(-1)
    kept = run(packed, packed)
    for a, b in zip(plain, kept):
        assert np.array_equal(a, b)
    # the buffer holds the bits of x > 0.5 (rows of whole words; what lies past the last frame's word is not specified)
    nw = (F + 31) // 32
    want = oracle.binarize_forward(host(x), F, 0.5, bit=True)
    assert np.array_equal(host(packed)[:, :nw], want[:, :nw])
    # the copy is what the backward call reads: with another input's bits in it the gradients change
    other = ops.packed_input_buffer(I, F)
    other.copy_(packed)
    other[:, :nw] ^= 0x55555555
    swapped = run(None, other)
    assert not np.array_equal(swapped[-1], plain[-1])
    # buffers that do not fit the call are ignored: another row count, a pitch that is not a multiple of eight words
    odd = torch.full((I, ((nw + 7) // 8) * 8 + 1), 0x33333333, dtype=torch.int32, device="cuda")
    again = run(odd, odd)
    for a, b in zip(plain, again):
        assert np.array_equal(a, b)
    assert int((odd != 0x33333333).sum()) == 0                          # and not written to


def test_the_hint_is_spent_by_the_next_entry(ops):
    """a packed copy offered before some other entry must not reach a later LUT call"""
    import torch
    from binarybrain_amd.capi import lib
    from binarybrain_amd.ops import ptr
    I, O, F = 40, 30, 256
    rng = np.random.default_rng(9)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S)); dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O)); rev = ops.reverse_table(idx, I)
    ops.set_dx_mode(0)
    dW0 = torch.zeros((O, 64), device="cuda"); dW1 = torch.zeros((O, 64), device="cuda")
    dx0 = ops.stochastic_lut_backward(6, x, dy, idx, W, dW0, F, rev, input_binary=True)
    junk = ops.packed_input_buffer(I, F); junk.fill_(0x0f0f0f0f)
    lib().bbhip_HintPackedInput(ptr(junk), I, junk.shape[1], 1)
    ops.hard_tanh_forward(x, F)                                         # any entry spends the hint
    dx1 = ops.stochastic_lut_backward(6, x, dy, idx, W, dW1, F, rev, input_binary=True)
    assert torch.equal(dx0, dx1) and torch.equal(dW0, dW1)
