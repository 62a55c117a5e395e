"""CPU suite: the C-ABI library loads without a GPU and exports every symbol include/bbhip.h declares; the ctypes
binding covers the same set; the host-side C++ plumbing passes its own test program."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bbhip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bbhip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from binarybrain_amd import capi
    from binarybrain_amd.build import LIB_PATH
    assert os.path.exists(LIB_PATH), "build the library first: python -m binarybrain_amd.build"
    lib = ctypes.CDLL(LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), "%s is declared in include/bbhip.h but not exported" % name
    assert sorted(capi.exported_symbols()) == names, "ctypes binding and header disagree"
    capi.lib()      # binds argument types of every symbol


def test_runtime_shim_without_gpu():
    from binarybrain_amd import capi
    lib = capi.lib()
    n = lib.bbhip_GetDeviceCount()
    assert n >= 0
    lib.bbhip_SetHostOnly(1)
    assert lib.bbhip_IsHostOnly() == 1 and lib.bbhip_IsDeviceAvailable() == 0
    lib.bbhip_SetHostOnly(0)
    assert lib.bbhip_IsDeviceAvailable() == (1 if n > 0 else 0)
    lib.bbhip_SetDxMode(2); assert lib.bbhip_GetDxMode() == 2
    lib.bbhip_SetDxMode(7); assert lib.bbhip_GetDxMode() == 0
    # argument checks come before any device work
    assert lib.bbhip_fp32_StochasticLut_Forward(9, None, None, None, None, 1, 1, 1, 0, 0, 0.25, None) != 0
    assert b"null buffer" in lib.bbhip_GetLastErrorString() or b"n=9" in lib.bbhip_GetLastErrorString()


def test_ops_fail_loudly_without_device_tensors():
    import torch
    from binarybrain_amd import ops
    from binarybrain_amd.capi import BbhipError
    x = torch.zeros((8, 64)); idx = torch.zeros((4, 6), dtype=torch.int32); W = torch.zeros((4, 64))
    with pytest.raises(BbhipError):
        ops.stochastic_lut_forward(6, x, idx, W, 64)


def test_host_side_cpp():
    exe = os.path.join(ROOT, "tests", "cpp", "test_host")
    if not os.path.exists(exe):
        from binarybrain_amd.build import build_cpp_tests
        build_cpp_tests()
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout


def test_binding_header_signatures():
    """include/bbcu_hip_binding.h gives every entry the reference's name and parameter list: tests/cpp/test_binding.cpp holds
    the reference's declarations (include/bbcu/bbcu.h) as function-pointer types and static_asserts each one, for the LUT
    widths 2..6; compiling it is the test, running it prints the count."""
    exe = os.path.join(ROOT, "tests", "cpp", "test_binding")
    if not os.path.exists(exe):
        from binarybrain_amd.build import build_cpp_tests
        build_cpp_tests()
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0 and "signatures equal the reference's declarations" in res.stdout, res.stdout
