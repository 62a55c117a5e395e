"""The kernels behind the environment switches.  The library reads its switches once per process, so each setting runs the
same parity case (tests/two_valued_case.py) in one child process: the default (lookup kernels for two-valued inputs,
packed backward pass) and the polynomial kernels for the same inputs."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("env", [{}, {"BBHIP_CORNER": "2", "BBHIP_PACK": "2"}, {"BBHIP_PACK": "2"}, {"BBHIP_CORNER": "0", "BBHIP_PACK": "0"},
                                 {"BBHIP_CORNER": "0"}, {"BBHIP_FWD_NODES": "1", "BBHIP_BWD_SLAB": "256"},
                                 {"BBHIP_DX_STEPS": "1", "BBHIP_DX_CHUNK": "64", "BBHIP_BIN_NODES": "1", "BBHIP_BIN_CHUNK": "64"},
                                 {"BBHIP_DX_STEPS": "4", "BBHIP_DX_CHUNK": "512", "BBHIP_FWD_CHUNK": "512", "BBHIP_BIN_NODES": "2", "BBHIP_BIN_CHUNK": "256"},
                                 {"BBHIP_DX_SPLIT": "1"}, {"BBHIP_DX_SPLIT": "0", "BBHIP_BIN_NODES": "4"},
                                 {"BBHIP_DX_WIDE": "0"}, {"BBHIP_INLINE_TABLES": "0"}, {"BBHIP_FWD_CHUNK": "2048"}, {"BBHIP_DX_INDEXED": "0"}, {"BBHIP_TERM_NODES": "0"}])
def test_two_valued_inputs_under_switches(env):
    child_env = dict(os.environ)
    child_env.update(env)
    child_env["PYTHONPATH"] = os.pathsep.join([os.path.dirname(HERE), HERE, child_env.get("PYTHONPATH", "")])
    p = subprocess.run([sys.executable, os.path.join(HERE, "two_valued_case.py")], env=child_env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0 and "two-valued case ok" in p.stdout, (env, p.stdout[-2000:], p.stderr[-2000:])
    # the switches took effect: 0 and 2 turn a path off, unset leaves it on
    want = {name: 0 if env.get(var) in ("0", "2") else 1 for name, var in (("corner", "BBHIP_CORNER"), ("pack", "BBHIP_PACK"))}
    assert "switches corner=%d pack=%d" % (want["corner"], want["pack"]) in p.stdout, (env, p.stdout[-500:])
