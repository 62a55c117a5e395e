"""The entry points under HIP graph capture: a DifferentiableLut6 layer's forward + backward and a StochasticLut6
forward + backward are captured once (through torch's capture stream; every entry point launches on the stream it is
given and, once its scratch arena has its size, calls nothing that a capture forbids) and replayed several times with
new contents in the same buffers, with eager work and synchronisations between the replays.  Every replay must equal the
eager result of the same inputs bit for bit: the default dx mode is deterministic."""
import numpy as np
import pytest

from binarybrain_amd import synth
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32


def _inputs(rng, I, O, F, stride):
    x = synth.uniform_frames(rng, I, F, stride)
    dy = synth.normal_frames(rng, O, F, stride)
    return x, dy


@pytest.mark.parametrize("layer", ["stochastic", "differentiable"])
def test_replays_equal_eager(layer):
    import torch
    from binarybrain_amd import ops
    ops.set_dx_mode(0)
    I, O, F = 96, 200, 700
    rng = np.random.default_rng(77)
    stride = synth.frame_stride_fp32(F)
    idx = dev(synth.wiring(rng, I, O))
    W = dev(synth.lut_tables(rng, O))
    rev = ops.reverse_table(idx, I)
    x, dy = (dev(a) for a in _inputs(rng, I, O, F, stride))
    dW = torch.zeros((O, 64), device="cuda")
    rm, rv = torch.zeros(O, device="cuda"), torch.ones(O, device="cuda")
    out = {}

    def step():
        dW.zero_()
        if layer == "stochastic":
            y = ops.stochastic_lut_forward(6, x, idx, W, F)
            dx = ops.stochastic_lut_backward(6, x, dy, idx, W, dW, F, rev)
        else:
            rm.zero_(); rv.fill_(1.0)
            y, mean, rstd = ops.differentiable_lut_forward_training(6, x, idx, W, F, rm, rv)
            dx = ops.differentiable_lut_backward(6, x, dy, idx, W, dW, F, mean, rstd, rev)
        out["y"], out["dx"] = y, dx

    def snapshot():
        torch.cuda.synchronize()
        return host(out["y"])[:, :F].copy(), host(out["dx"])[:, :F].copy(), host(dW).copy(), host(rm).copy(), host(rv).copy()

    step(); step()                                   # the arena reaches its size before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    graph_out = dict(out)

    for k in range(4):
        xh, dyh = _inputs(rng, I, O, F, stride)
        x.copy_(dev(xh)); dy.copy_(dev(dyh))
        step()                                       # eager, into fresh output tensors
        want = snapshot()
        out.update(graph_out)
        dW.fill_(123.0)                              # the replay must redo the zeroing it captured
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for a, b, name in zip(got, want, ("y", "dx", "dW", "running_mean", "running_var")):
            assert np.array_equal(a, b), (layer, k, name)
        assert np.abs(got[1]).max() > 0 and np.abs(got[2]).max() > 0


def test_replay_survives_arena_growth_and_capture_refuses_to_grow():
    """A graph captured at one size keeps replaying correctly after a larger eager call has made the scratch arena grow
    (the outgrown block stays allocated), and a call that would have to grow the arena during a capture fails with a
    message instead of allocating under the capture."""
    import torch
    from binarybrain_amd import capi, ops
    ops.set_dx_mode(0)
    capi.check(capi.lib().bbhip_ReleaseScratch())
    I, O, F = 64, 96, 300
    rng = np.random.default_rng(5)
    stride = synth.frame_stride_fp32(F)
    idx = dev(synth.wiring(rng, I, O)); W = dev(synth.lut_tables(rng, O)); rev = ops.reverse_table(idx, I)
    x, dy = (dev(a) for a in _inputs(rng, I, O, F, stride))
    dW = torch.zeros((O, 64), device="cuda")
    out = {}

    def step():
        dW.zero_()
        out["y"] = ops.stochastic_lut_forward(6, x, idx, W, F)
        out["dx"] = ops.stochastic_lut_backward(6, x, dy, idx, W, dW, F, rev)

    step(); torch.cuda.synchronize()
    small = capi.lib().bbhip_GetScratchSize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    graph_out = dict(out)

    # a larger layer: the arena grows, its old block must stay valid for the graph
    I2, O2, F2 = 256, 4096, 2048
    s2 = synth.frame_stride_fp32(F2)
    idx2 = dev(synth.wiring(rng, I2, O2)); W2 = dev(synth.lut_tables(rng, O2)); rev2 = ops.reverse_table(idx2, I2)
    x2 = dev(synth.uniform_frames(rng, I2, F2, s2)); dy2 = dev(synth.normal_frames(rng, O2, F2, s2))
    dW2 = torch.zeros((O2, 64), device="cuda")
    ops.stochastic_lut_forward(6, x2, idx2, W2, F2)
    ops.stochastic_lut_backward(6, x2, dy2, idx2, W2, dW2, F2, rev2)
    torch.cuda.synchronize()
    assert capi.lib().bbhip_GetScratchSize() > small

    for k in range(2):
        xh, dyh = _inputs(rng, I, O, F, stride)
        x.copy_(dev(xh)); dy.copy_(dev(dyh))
        step(); torch.cuda.synchronize()
        want = (host(out["y"]).copy(), host(out["dx"]).copy(), host(dW).copy())
        out.update(graph_out)
        graph.replay(); torch.cuda.synchronize()
        got = (host(out["y"]), host(out["dx"]), host(dW))
        for a, b, name in zip(got, want, ("y", "dx", "dW")):
            assert np.array_equal(a[:, :F] if name != "dW" else a, b[:, :F] if name != "dW" else b), (k, name)

    # growth under capture is refused
    del graph
    capi.check(capi.lib().bbhip_ReleaseScratch())
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(capi.BbhipError, match="stream capture"):
        with torch.cuda.graph(g2):
            ops.stochastic_lut_forward(6, x, idx, W, F)
    torch.cuda.synchronize()
    # reserving first makes the same capture legal
    capi.check(capi.lib().bbhip_ReserveScratch(1 << 22))
    g3 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g3):
        y3 = ops.stochastic_lut_forward(6, x, idx, W, F)
    g3.replay(); torch.cuda.synchronize()
    assert np.array_equal(host(y3)[:, :F], host(ops.stochastic_lut_forward(6, x, idx, W, F))[:, :F])
