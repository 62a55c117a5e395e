"""Builds binarybrain_amd/lib/libbbhip.so (hand-written HIP kernels + the C ABI) for gfx950 with hipcc."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbbhip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU instructions are disabled on purpose: scalar fp32 code must not be auto-vectorised into v_pk_* forms
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-munsafe-fp-atomics",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC] + FLAGS + [os.path.join(CSRC, "bbhip.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 target feature; that is expected
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
