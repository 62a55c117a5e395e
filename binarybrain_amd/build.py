"""Builds binarybrain_amd/lib/libbbhip.so (hand-written HIP kernels + the C ABI) for gfx950 with hipcc, and the
C++ programs that exercise the host-side model classes."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbbhip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU instructions are disabled on purpose: scalar fp32 code must not be auto-vectorised into v_pk_* forms
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-munsafe-fp-atomics",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 target feature; that is expected
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    if verbose and out.strip():
        print(out)


def build_library(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    _run([HIPCC] + FLAGS + [os.path.join(CSRC, "bbhip.hip"), "-o", LIB_PATH], verbose)
    return LIB_PATH


def build_bench_probe(verbose=False):
    """bench_gather_probe.so beside bench.py: the instrumentation kernel of `bench.py --workload gather_ceiling` (not part of the library)."""
    out = os.path.join(ROOT, "bench_gather_probe.so")
    _run([HIPCC] + FLAGS + ["-I" + ROOT, os.path.join(ROOT, "bench_gather_probe.hip"), "-o", out], verbose)
    return out


def build_cpp_tests(verbose=False):
    """tests/cpp/test_host, object_tool and test_binding (CPU; test_binding --gpu runs on the device) and tests/cpp/test_models
    (GPU): plain host C++ over the C ABI; the oracle library is linked as the checker."""
    out = []
    for name in ("test_host", "test_models", "object_tool", "test_binding"):
        exe = os.path.join(ROOT, "tests", "cpp", name)
        _run(["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "include"),
              os.path.join(ROOT, "tests", "cpp", name + ".cpp"), "-o", exe,
              "-L" + LIB_DIR, "-lbbhip", "-L" + os.path.join(ROOT, "oracle"), "-loracle",
              "-Wl,-rpath,$ORIGIN/../../binarybrain_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"], verbose)
        out.append(exe)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
