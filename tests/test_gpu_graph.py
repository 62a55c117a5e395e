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
