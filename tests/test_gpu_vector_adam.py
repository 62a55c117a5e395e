"""GPU parity of the elementwise vector operations and the Adam step (through the C ABI) against the CPU oracle.
Every operation is individually rounded on both sides, so the bar is bit-exact, except exp (library function on both
sides: 2 ulp)."""
import os

import numpy as np
import pytest

import oracle
from util import dev, host

pytestmark = pytest.mark.gpu
F32 = np.float32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "adam.npz"))


@pytest.fixture(scope="module")
def ops():
    from binarybrain_amd import ops as o
    return o


def _ulp_close(a, b, ulps):
    tol = ulps * np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(F32))
    return bool(np.all(np.abs(a.astype(np.float64) - b.astype(np.float64)) <= tol))


@pytest.mark.parametrize("size", [1, 3, 4, 1023, 4096, 1 << 20, (1 << 20) + 5])
def test_vector_ops(ops, size):
    rng = np.random.default_rng(size)
    x = (rng.standard_normal(size) * 3).astype(F32); y = (rng.standard_normal(size) * 3).astype(F32)
    pos = np.abs(y) + F32(0.5)
    dx, dy_, dpos = dev(x), dev(y), dev(pos)
    a, b, c, d = 1.25, -0.6, 0.3, 2.0
    assert np.array_equal(host(ops.vector_add_ex(dx, dy_, a, b, c)), oracle.vector_op("add_ex", x, y, a, b, c))
    assert np.array_equal(host(ops.vector_mul_ex(dx, dy_, a, b)), oracle.vector_op("mul_ex", x, y, a, b))
    assert np.array_equal(host(ops.vector_div_ex(dx, dpos, a, b, c, d)), oracle.vector_op("div_ex", x, pos, a, b, c, d))
    assert np.array_equal(host(ops.vector_unary("sqrt", dpos)), oracle.vector_op("sqrt", pos))
    assert _ulp_close(host(ops.vector_unary("exp", dx)), oracle.vector_op("exp", x), 2)
    assert np.array_equal(host(ops.vector_minmax("min", dx, dy_)), oracle.vector_op("min", x, y))
    assert np.array_equal(host(ops.vector_minmax("max", dx, dy_)), oracle.vector_op("max", x, y))
    assert np.array_equal(host(ops.vector_minmax("min", dx, 0.4)), oracle.vector_op("min_v", x, None, 0.4))
    assert np.array_equal(host(ops.vector_minmax("max", dx, 0.4)), oracle.vector_op("max_v", x, None, 0.4))
    # in place, and through a view that is not 16-byte aligned
    if size > 8:
        t = dev(x.copy())
        ops.vector_add_ex(t, dy_, 1.0, 1.0, 0.0, out=t)
        assert np.array_equal(host(t), x + y)
        v = dev(x)[1:]; w = dev(y)[1:]
        assert np.array_equal(host(ops.vector_mul_ex(v, w, 2.0, 1.0)), oracle.vector_op("mul_ex", x[1:], y[1:], 2.0, 1.0))


def test_vector_ops_reference_vectors(ops):
    x, y, pos = GOLD["vx"], GOLD["vy"], GOLD["vpos"]
    assert np.array_equal(host(ops.vector_unary("sqrt", dev(pos))), GOLD["sqrt"])
    assert np.array_equal(host(ops.vector_minmax("min", dev(x), dev(y))), GOLD["min"])
    assert np.array_equal(host(ops.vector_minmax("max", dev(x), 0.3)), GOLD["max_v"])
    n = np.array([np.nan, 1.0], F32); o = np.array([1.0, np.nan], F32)
    r = host(ops.vector_minmax("min", dev(n), dev(o)))
    assert np.isnan(r[0]) and r[1] == 1.0


def test_adam_reference_vectors(ops):
    import torch
    for k in range(int(GOLD["adam_count"][0])):
        lr, b1, b2 = GOLD["a%d_hyper" % k]
        p = dev(GOLD["a%d_p0" % k].copy()); g = torch.zeros_like(p)
        st = ops.AdamState([p], [g], lr, b1, b2)
        for gt in GOLD["a%d_g" % k]:
            g.copy_(dev(gt))
            st.step()
        assert np.array_equal(host(p), GOLD["a%d_p" % k]), k


def test_adam_many_tensors(ops):
    """A parameter list shaped like the benchmark network's (three LUT layers: W tables of 6144, 1024 and 70 nodes)."""
    import torch
    rng = np.random.default_rng(3)
    shapes = [(6144, 64), (1024, 64), (70, 64), (1,), (5,)]
    p0 = [rng.random(s).astype(F32) for s in shapes]
    params = [dev(a.copy()) for a in p0]
    grads = [torch.zeros_like(p) for p in params]
    st = ops.AdamState(params, grads, 0.001, 0.9, 0.999)
    gs = [[(rng.standard_normal(s) * 0.1).astype(F32) for s in shapes] for _ in range(4)]
    for step in gs:
        for g, a in zip(grads, step):
            g.copy_(dev(a))
        st.step()
    for i, s in enumerate(shapes):
        ref, m, v = oracle.adam_steps(p0[i].ravel(), [step[i].ravel() for step in gs], 0.001, 0.9, 0.999)
        assert np.array_equal(host(params[i]).ravel(), ref), s
        assert np.array_equal(host(st.m[i]).ravel(), m) and np.array_equal(host(st.v[i]).ravel(), v)


def test_adam_update_is_step_then_zero_grad(ops):
    """bbhip_fp32_OptimizerAdam_Update = the optimizer's Update(): Step() followed by ZeroGrad() (include/bb/Optimizer.h:31-35).
    Parameters and moments equal those of the plain step bit for bit, and every gradient element is zero afterwards; tensor
    sizes include ones that are not a multiple of four and pointers that are not 16-byte aligned (the scalar tail of the kernel)."""
    import torch
    rng = np.random.default_rng(11)
    shapes = [(1024, 64), (70, 64), (1,), (5,), (1031,)]
    p0 = [rng.random(s).astype(F32) for s in shapes]
    gs = [[(rng.standard_normal(s) * 0.1).astype(F32) for s in shapes] for _ in range(3)]
    out = {}
    for mode in ("step", "update"):
        backing = [torch.zeros(int(np.prod(s)) + 1, device="cuda") for s in shapes]
        params = [dev(a.copy()) for a in p0]
        grads = [b[1:].view(*s) if i == 4 else b[:-1].view(*s) for i, (b, s) in enumerate(zip(backing, shapes))]      # the last one misaligned
        st = ops.AdamState(params, grads, 0.001, 0.9, 0.999)
        for step in gs:
            for g, a in zip(grads, step):
                g.copy_(dev(a))
            if mode == "step":
                st.step()
                assert all(np.array_equal(host(g), a) for g, a in zip(grads, step))       # the plain step leaves the gradients alone
            else:
                st.update()
                assert all(not host(g).any() for g in grads)
        out[mode] = ([host(p) for p in params], [host(m) for m in st.m], [host(v) for v in st.v])
    for a, b in zip(out["step"], out["update"]):
        assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_rejects_bad_arguments(ops):
    from binarybrain_amd import capi
    import ctypes as C
    lib = capi.lib()
    assert lib.bbhip_fp32_Vector_sqrt(None, None, 4, None) != 0
    assert b"rejected" in lib.bbhip_GetLastErrorString()
    assert lib.bbhip_fp32_Vector_add_ex(None, None, None, 1.0, 1.0, 0.0, 0, None) != 0
    assert lib.bbhip_fp32_OptimizerAdam(-1, None, None, None, None, None, 0.1, 0.9, 0.999, None) != 0
    assert lib.bbhip_fp32_OptimizerAdam(0, None, None, None, None, None, 0.1, 0.9, 0.999, None) == 0
