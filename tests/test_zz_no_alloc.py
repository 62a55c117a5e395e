"""bbhip_fp32_StochasticLut_Forward_NoAlloc (the entry point that allocates nothing) against bbhip_fp32_StochasticLut_Forward,
through the C ABI: two calls in a row, the second on a smaller layer, so that the fixed scratch block still holds the first
call's tables when the second runs; then a layer beyond the block's size, which must be rejected with a message."""
import numpy as np
import pytest

from binarybrain_amd import capi, synth
from binarybrain_amd.capi import check, lib, ptr, stream_ptr
from util import dev, host

pytestmark = pytest.mark.gpu


def _forward(entry, n, x, idx, W, y, O, F, stride, input_binary, lut_binarize):
    import torch
    check(getattr(lib(), entry)(n, ptr(x), ptr(y), ptr(idx), ptr(W), O, F, stride, input_binary, lut_binarize, 0.25, stream_ptr()))
    torch.cuda.synchronize()
    return host(y)


@pytest.mark.parametrize("input_binary,lut_binarize", [(0, 0), (1, 0), (0, 1)])
def test_no_alloc_forward_equals_forward(input_binary, lut_binarize):
    import torch
    rng = np.random.default_rng(31 + input_binary + 2 * lut_binarize)
    for n, I, O, F in ((6, 300, 2000, 1100), (6, 64, 70, 130), (4, 50, 33, 64)):      # second and third calls: smaller layers
        stride = synth.frame_stride_fp32(F)
        idx = dev(synth.wiring(rng, I, O, n)); W = dev(synth.lut_tables(rng, O, n))
        x = dev(synth.uniform_frames(rng, I, F, stride, -0.1, 1.1))
        y_got = torch.full((O, stride), -7.0, device="cuda"); y_want = torch.full((O, stride), -7.0, device="cuda")
        # The call must allocate nothing: with the library's own scratch arena given back first, it may not grow it again, and the
        # device's free memory is the same after the call as before (the outputs were allocated above).
        capi.check(lib().bbhip_fp32_Vector_set(ptr(y_want), -7.0, 1, stream_ptr()))     # (in a fresh process: the library's code is loaded by its first launch)
        torch.cuda.synchronize()
        check(lib().bbhip_ReleaseScratch())
        assert lib().bbhip_GetScratchSize() == 0
        free_before = torch.cuda.mem_get_info()[0]
        got = _forward("bbhip_fp32_StochasticLut_Forward_NoAlloc", n, x, idx, W, y_got, O, F, stride, input_binary, lut_binarize)
        assert lib().bbhip_GetScratchSize() == 0, "the entry that allocates nothing grew the scratch arena"
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated during the call"
        want = _forward("bbhip_fp32_StochasticLut_Forward", n, x, idx, W, y_want, O, F, stride, input_binary, lut_binarize)
        assert lib().bbhip_GetScratchSize() > 0                       # (the arena path does use the arena)
        # same kernels, same tables: identical bits (with input_binary the arena path may pack the input first when it is
        # told the row count; it is not told here)
        assert np.array_equal(got[:, :F], want[:, :F]), (n, I, O, F)
        assert np.all(got[:, F:] == -7.0)


def test_no_alloc_forward_rejects_layers_beyond_its_block():
    import torch
    n, O, F = 6, 40000, 64              # 40000 * 64 * 4 bytes > 8 MiB
    x = torch.zeros((8, 64), device="cuda"); y = torch.zeros((O, 64), device="cuda")
    idx = torch.zeros((O, 6), dtype=torch.int32, device="cuda"); W = torch.zeros((O, 64), device="cuda")
    rc = lib().bbhip_fp32_StochasticLut_Forward_NoAlloc(n, ptr(x), ptr(y), ptr(idx), ptr(W), O, F, 64, 0, 0, 0.25, stream_ptr())
    assert rc != 0 and b"fixed block" in lib().bbhip_GetLastErrorString()
    # the arena path takes the same layer
    check(lib().bbhip_fp32_StochasticLut_Forward(n, ptr(x), ptr(y), ptr(idx), ptr(W), O, F, 64, 0, 0, 0.25, stream_ptr()))
    torch.cuda.synchronize()
