"""GPU: the C++ model classes (bb::StochasticLutN / DifferentiableLutN / BinaryLutN over the C ABI) against the oracle.
The program is built beforehand by __graft_entry__.build(); its source is tests/cpp/test_models.cpp."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_model_classes():
    exe = os.path.join(ROOT, "tests", "cpp", "test_models")
    assert os.path.exists(exe), "tests/cpp/test_models is missing: run __graft_entry__.build()"
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout)
    assert res.returncode == 0, res.stdout


def test_layer_through_the_reference_named_binding():
    """One StochasticLut6 forward + backward called through the templates of include/bbcu_hip_binding.h (the reference's
    names, default width and default stream) equals the same calls on the C ABI bit for bit; a rejected call throws."""
    exe = os.path.join(ROOT, "tests", "cpp", "test_binding")
    assert os.path.exists(exe), "tests/cpp/test_binding is missing: run __graft_entry__.build()"
    res = subprocess.run([exe, "--gpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout)
    assert res.returncode == 0, res.stdout
