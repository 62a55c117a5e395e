"""profiles/traffic.json (HBM-side bytes from hardware counters, written by `bench.py --write-traffic`) is what the bench line's
`roofline.traffic` reports: the file has the kernels the bench names, the helper reads them, and the hash on the line is the file's
git blob hash."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_traffic_file_feeds_the_bench_line():
    data = json.load(open(bench.TRAFFIC_FILE))
    for name in ("stochasticlut6/lut_dx_kernel", "stochasticlut6/lut_forward_kernel", "stochasticlut6/lut_backward_kernel",
                 "binarylut6/binary_lut6_kernel", "adam/adam_kernel"):
        entry = data["kernels"][name]
        assert entry["bytes"] == entry["fetch_bytes"] + entry["write_bytes"] > 0
        assert bench.measured_traffic("kernels", name) == entry["bytes"]
    for name in ("mnist_step", "conv_block"):
        assert bench.measured_traffic("steps", name) == data["steps"][name]["bytes"] > 0
    assert bench.measured_traffic("kernels", "no such kernel") is None
    # the counter units come from a plain copy of known size: 2 KiB per FETCH_SIZE count, 1 KiB per WRITE_SIZE count on this GPU
    assert abs(data["counter_unit_bytes"]["FETCH_SIZE"] / 2048.0 - 1.0) < 0.01 and abs(data["counter_unit_bytes"]["WRITE_SIZE"] / 1024.0 - 1.0) < 0.01
    # HBM traffic is never below what the algorithm must move
    assert data["kernels"]["stochasticlut6/lut_dx_kernel"]["bytes"] >= 4 * 8192 * (2 * 4096 + 4096)
    # the commands that make the file run committed files only
    assert all("bench.py" in c for c in data["made_by"]) and data["made_by"] == bench.TRAFFIC_COMMANDS


def test_hash_on_the_bench_line_is_the_git_blob_hash():
    src = bench.traffic_source()
    assert src["file"] == "profiles/traffic.json" and len(src["git_blob"]) == 40
    try:
        want = subprocess.run(["git", "hash-object", bench.TRAFFIC_FILE], cwd=ROOT, capture_output=True, text=True, timeout=30)
    except (OSError, subprocess.TimeoutExpired):
        return
    if want.returncode == 0:
        assert src["git_blob"] == want.stdout.strip()
