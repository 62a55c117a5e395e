"""The caller-owned copy of the tables that a LUT call derives from W (bbhip_HintPreparedTables): the forward call of a step writes
them into the caller's buffer, the backward call of the same step reads them there instead of preparing them again, and neither
changes a bit of any result; a buffer that does not fit the call is ignored."""
import numpy as np
import pytest

from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _frames(t, F, S):
    a = host(t)
    return a[:, :F] if a.ndim == 2 and a.shape[1] == S else a           # what lies past the last frame of a row is not specified


@pytest.mark.parametrize("n", [6, 4, 2])
@pytest.mark.parametrize("shape", [(64, 48, 1024), (27, 216, 5000), (784, 300, 200), (100, 70, 37)])
@pytest.mark.parametrize("kind", ["fp32_binary", "fp32_real", "bit"])
@pytest.mark.parametrize("lut_binarize", [False, True])
def test_results_do_not_depend_on_the_kept_tables(ops, n, shape, kind, lut_binarize):
    import torch
    I, O, F = shape
    rng = np.random.default_rng(I + O + F + n)
    S = synth.frame_stride_fp32(F)
    dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O, n))
    W = dev(synth.lut_tables(rng, O, n))
    rev = ops.reverse_table(idx, I)
    ops.set_dx_mode(0)
    x = dev(synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))) if kind == "bit" else dev(synth.uniform_frames(rng, I, F, S))

    def run(tables, with_packed=False):
        dW = torch.zeros((O, 1 << n), device="cuda")
        rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
        if kind == "bit":
            y, mean, rstd = ops.bit_differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize, tables=tables)
            dx = ops.bit_differentiable_lut_backward(n, x, dy, idx, W, dW, F, mean, rstd, rev, lut_binarize=lut_binarize, tables=tables)
        else:
            packed = ops.packed_input_buffer(I, F) if with_packed else None
            binary = kind == "fp32_binary"
            y, mean, rstd = ops.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, lut_binarize=lut_binarize, binary_mode=binary,
                                                                    packed=packed, tables=tables)
            dx = ops.differentiable_lut_backward(n, x, dy, idx, W, dW, F, mean, rstd, rev, lut_binarize=lut_binarize, binary_mode=binary,
                                                 packed=packed, tables=tables)
        return [_frames(t, F, S) for t in (y, mean, rstd, rm, rv, dx, dW)]

    plain = run(None)
    tables = ops.prepared_tables_buffer(n, O)
    tables.fill_(float("nan"))
    for a, b in zip(plain, run(tables)):
        assert np.array_equal(a, b)
    assert not np.isnan(host(tables)[:O * (1 << n)]).any()              # the forward call wrote the coefficients there
    if kind == "fp32_binary":
        for a, b in zip(plain, run(tables, with_packed=True)):          # together with the kept packed copy of the input
            assert np.array_equal(a, b)


def test_the_backward_call_reads_the_kept_tables(ops):
    """with other tables in the buffer the gradients change: the buffer is what the call uses"""
    import torch
    I, O, F, n = 64, 48, 1024, 6
    rng = np.random.default_rng(3)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S)); dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O)); other = dev(synth.lut_tables(rng, O))
    rev = ops.reverse_table(idx, I)
    rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
    tables = ops.prepared_tables_buffer(n, O)
    y, mean, rstd = ops.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, tables=tables)
    dW0 = torch.zeros((O, 64), device="cuda"); dW1 = torch.zeros((O, 64), device="cuda"); dW2 = torch.zeros((O, 64), device="cuda")
    dx0 = ops.differentiable_lut_backward(n, x, dy, idx, W, dW0, F, mean, rstd, rev)
    dx1 = ops.differentiable_lut_backward(n, x, dy, idx, W, dW1, F, mean, rstd, rev, tables=tables)
    assert torch.equal(dx0[:, :F], dx1[:, :F]) and torch.equal(dW0, dW1)
    ops.differentiable_lut_forward_training(n, x, idx, other, F, rm.clone(), rv.clone(), tables=tables)      # another layer's tables
    ops.differentiable_lut_backward(n, x, dy, idx, W, dW2, F, mean, rstd, rev, tables=tables)
    assert not torch.equal(dW0, dW2)


def test_a_buffer_that_does_not_fit_is_ignored(ops):
    import torch
    I, O, F, n = 64, 48, 300, 6
    rng = np.random.default_rng(4)
    S = synth.frame_stride_fp32(F)
    x = dev(synth.uniform_frames(rng, I, F, S)); dy = dev(synth.normal_frames(rng, O, F, S))
    idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O))
    rev = ops.reverse_table(idx, I)

    def run(tables):
        rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
        dW = torch.zeros((O, 64), device="cuda")
        y, mean, rstd = ops.differentiable_lut_forward_training(n, x, idx, W, F, rm, rv, tables=tables)
        dx = ops.differentiable_lut_backward(n, x, dy, idx, W, dW, F, mean, rstd, rev, tables=tables)
        return [_frames(t, F, S) for t in (y, mean, rstd, dx, dW)]

    plain = run(None)
    small = torch.full((O * 64,), -7.0, device="cuda")                  # half of what the call needs
    shifted = torch.full((2 * O * 64 + 256,), -7.0, device="cuda")[1:]  # large enough, not 256-byte aligned
    for buf in (small, shifted):
        for a, b in zip(plain, run(buf)):
            assert np.array_equal(a, b)
        assert (host(buf) == -7.0).all()                                # and not written to
    assert ops.lib().bbhip_PreparedTablesBytes(6, 48) == 2 * 48 * 64 * 4 and ops.lib().bbhip_PreparedTablesBytes(7, 48) == 0
