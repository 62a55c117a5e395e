"""Helpers shared by the GPU parity tests."""
import numpy as np

FWD_TOL = 1e-5     # |gpu - oracle| <= FWD_TOL * max(1, |oracle|): fp32 forward (values live in [0, 1])
BWD_TOL = 1e-4     # max|gpu - oracle| <= BWD_TOL * max|oracle|: dW and dx (accumulation order differs)


def rel_err(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def assert_fwd(gpu, ref, what=""):
    gpu = np.asarray(gpu, np.float64); ref = np.asarray(ref, np.float64)
    err = np.abs(gpu - ref) / np.maximum(1.0, np.abs(ref))
    assert err.max() <= FWD_TOL, "%s forward err %.3g" % (what, err.max())


def assert_bwd(gpu, ref, what=""):
    e = rel_err(gpu, ref)
    assert e <= BWD_TOL, "%s backward rel err %.3g" % (what, e)


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()
