"""Benchmark of the differentiable-LUT hot path on one MI355X.

A step is one pass of StochasticLut6 over one batch of synthetic input: clamp W, forward, backward (dW and dx), fp32,
4096 input nodes -> 4096 output nodes, 8192 frames.  Inputs are resident in HBM before the timed region.
Prints ONE JSON line: node-evaluations per second (one node-eval = one (output node, frame) pair taken through forward
and backward), the HBM roofline of the dominant kernel, and the CPU reference timed on this host's cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E peak, GB/s

# HBM-side bytes per launch (per step, for the step workloads) come from the hardware counters FETCH_SIZE and WRITE_SIZE, collected with
# rocprofv3 and written to profiles/traffic.json by `bench.py --write-traffic` (TRAFFIC_COMMANDS below); nothing is measured twice
# here: the bench line carries what that file holds for the kernel, and the file's git blob hash, or null where the file has no entry.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
TRAFFIC_WORKLOADS = {          # workload -> (extra bench arguments, kernel that runs once per step)
    "stochasticlut6": ("--no-configs --profile-copy", "lut_dx_kernel"),
    "binarylut6": ("--profile-copy", "binary_lut6_kernel"),
    "adam": ("", "adam_kernel"),
    "mnist_step": ("", "adam_kernel"),
    "conv_block": ("", "im2col_backward_kernel"),
}
def traffic_commands(dirname="traffic_runs"):
    """the counter runs behind profiles/traffic.json (one counter per run), then the call that writes the file from them"""
    runs = ["rocprofv3 --pmc %s -d %s/%s/%s -o r -- python3 bench.py --workload %s --steps 5 --warmup 5 --ramp-seconds 0 --no-cpu %s"
            % (counter, dirname, w, counter, w, extra) for w, (extra, _) in TRAFFIC_WORKLOADS.items() for counter in ("FETCH_SIZE", "WRITE_SIZE")]
    return runs + ["python3 bench.py --write-traffic %s" % dirname]


TRAFFIC_COMMANDS = traffic_commands()


def _git_blob_hash(path):
    import hashlib
    data = open(path, "rb").read()
    return hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest()


_traffic_cache = None


def measured_traffic(section, name):
    """bytes from profiles/traffic.json: section "kernels" (per launch) or "steps" (per step); None when the file has no such entry"""
    global _traffic_cache
    if _traffic_cache is None:
        try:
            _traffic_cache = json.load(open(TRAFFIC_FILE))
            _traffic_cache["git_blob"] = _git_blob_hash(TRAFFIC_FILE)
        except (OSError, ValueError):
            _traffic_cache = {}
    entry = _traffic_cache.get(section, {}).get(name)
    return None if entry is None else entry["bytes"]


def traffic_source():
    measured_traffic("kernels", "")
    return {"file": "profiles/traffic.json", "git_blob": _traffic_cache.get("git_blob")}


def _short_kernel_name(name):
    """'void bbhip::lut_dx_kernel<6, 0, 2>(bbhip::DxArgs)' -> 'lut_dx_kernel'"""
    name = name.split("(")[0].replace("void ", "").strip()
    return name.split("<")[0].split("::")[-1]


def write_traffic(dirname):
    """Reads the counter runs of TRAFFIC_COMMANDS under `dirname` (rocprofv3's r_results.db per workload and counter) and writes
    profiles/traffic.json: per kernel of the library the mean FETCH_SIZE / WRITE_SIZE per dispatch in bytes, per step workload the sum
    over one step.  A counter's unit is taken from what it reads for the plain device copies of known size at the end of the
    `--profile-copy` runs (torch's copy kernel: x.numel() * 4 bytes read and as many written per copy)."""
    import sqlite3

    def counters(workload, counter):
        db = os.path.join(dirname, workload, counter, "r_results.db")
        con = sqlite3.connect(db)
        rows = con.execute("select kernel_name, value from counters_collection where counter_name = ? order by dispatch_id", (counter,)).fetchall()
        con.close()
        by = {}
        for name, value in rows:
            by.setdefault(name, []).append(float(value))
        return by

    copy_bytes = {"stochasticlut6": 4096 * 8320 * 4, "binarylut6": 8192 * 8288 * 4}
    unit = {}
    calibration = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        units = []
        for w, nbytes in copy_bytes.items():
            by = counters(w, counter)
            copies = [v for name, vals in by.items() if "copybuffer" in name.lower() for v in vals[-3:]]      # torch's device-to-device copy
            if copies:
                units.append(nbytes / (sum(copies) / len(copies)))
                calibration["%s, %s" % (counter, w)] = {"copy_bytes": nbytes, "counter_per_copy": sum(copies) / len(copies)}
        unit[counter] = sum(units) / len(units)
    out = {"made_by": TRAFFIC_COMMANDS, "counter_unit_bytes": unit, "calibration": calibration, "kernels": {}, "steps": {}}
    for w, (_, marker) in TRAFFIC_WORKLOADS.items():
        fetch, write = counters(w, "FETCH_SIZE"), counters(w, "WRITE_SIZE")
        steps = max(len(v) for name, v in fetch.items() if marker in name)
        step_bytes = 0.0
        for name in fetch:
            if "bbhip::" not in name:
                continue
            f = sum(fetch[name]) / len(fetch[name]) * unit["FETCH_SIZE"]
            wr = sum(write.get(name, [0.0])) / max(1, len(write.get(name, [0.0]))) * unit["WRITE_SIZE"]
            step_bytes += (f + wr) * len(fetch[name]) / steps
            if w in ("stochasticlut6", "binarylut6", "adam"):
                out["kernels"]["%s/%s" % (w, _short_kernel_name(name))] = {"bytes": f + wr, "fetch_bytes": f, "write_bytes": wr, "dispatches": len(fetch[name]), "workload": w}
        out["steps"][w] = {"bytes": step_bytes, "steps_counted": steps}
    with open(TRAFFIC_FILE, "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print("wrote %s: %d kernels, %d step workloads" % (TRAFFIC_FILE, len(out["kernels"]), len(out["steps"])))


def algorithmic_bytes(I, O, F):
    """every tensor touched once per pass, index and table traffic included (fp32, N = 6)"""
    fwd = 4 * F * (I + O) + 256 * O + 24 * O
    bwd = 4 * F * (2 * I + O) + 3 * 256 * O + 24 * O
    return fwd, bwd


def cpu_baseline(I, O, frames, threads, reps=9):
    """Forward+backward of the same layer on the host cores: the reference's own AVX2/OpenMP path when oracle/_ref is
    present ("reference"), else the C restatement ("port").  Timed around Forward+Backward only; median of reps."""
    import numpy as np
    os.environ["OMP_NUM_THREADS"] = str(threads)
    import oracle
    from binarybrain_amd import synth
    rng = np.random.default_rng(1)
    idx = synth.wiring(rng, I, O)
    W = synth.lut_tables(rng, O)
    x = synth.uniform_frames(rng, I, frames, frames)
    dy = synth.normal_frames(rng, O, frames, frames)
    secs, kind = oracle.time_stochastic_lut6(x, dy, idx, W, reps)
    med = float(np.median(secs))
    out = {"value": O * frames / med / 1e9, "unit": "G node-evals/s", "cores": threads, "kind": kind,
           "sample": "StochasticLut6 fwd+bwd (AVX2+OpenMP host path), %d->%d nodes, %d frames, 1 warm-up + median of %d"
                     % (I, O, frames, reps)}
    # the same code on one thread, on an eighth of the frames (the OpenMP thread count is switched through the runtime the
    # libraries share; the environment variable was read when it was loaded)
    try:
        import ctypes
        gomp = ctypes.CDLL("libgomp.so.1")
        gomp.omp_set_num_threads(1)
        f1 = max(64, frames // 8)
        secs1, _ = oracle.time_stochastic_lut6(np.ascontiguousarray(x[:, :f1]), np.ascontiguousarray(dy[:, :f1]), idx, W, 3)
        gomp.omp_set_num_threads(threads)
        out["value_1_thread"] = O * f1 / float(np.median(secs1)) / 1e9
        out["sample_1_thread"] = "%d frames, 1 warm-up + median of 3" % f1
    except OSError:
        pass
    try:
        with open("/proc/cpuinfo") as f:
            models = [l.split(":", 1)[1].strip() for l in f if l.startswith("model name")]
        out["cpu_model"] = models[0] if models else None
        out["host_logical_cpus"] = len(models)
    except OSError:
        pass
    return out


def bench_adam(args, lib):
    """One Adam update of a parameter list (secondary measurement): the three W tables of the MNIST-shaped LUT network
    (6144, 1024 and 70 nodes x 64 entries) followed by four 16 Mi-element tensors, so that the call is bandwidth-bound.
    Algorithmic bytes: 28 per element (read p, g, m, v; write p, m, v)."""
    import numpy as np
    import torch
    from binarybrain_amd import ops
    sizes = [6144 * 64, 1024 * 64, 70 * 64] + [1 << 24] * 4
    g = torch.Generator(device="cuda"); g.manual_seed(0)
    params = [torch.rand(n, device="cuda", generator=g) for n in sizes]
    grads = [torch.randn(n, device="cuda", generator=g) * 0.1 for n in sizes]
    st = ops.AdamState(params, grads)
    for _ in range(args.warmup):
        st.step()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        st.step()
    e1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    kernel_ms = e0.elapsed_time(e1) / args.steps          # back-to-back launches of the one kernel on the current stream
    total = sum(sizes)
    gbs = 28.0 * total / (kernel_ms * 1e-3) / 1e9
    out = {"metric": "G parameter updates/s, Adam fp32", "value": total / (dt / args.steps) / 1e9, "unit": "G updates/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "Adam step over %d tensors, %d elements" % (len(sizes), total)},
           "roofline": {"bound": "hbm", "kernel": "adam_kernel", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": gbs / HBM_PEAK_GBS, "traffic": measured_traffic("kernels", "adam/adam_kernel"), "traffic_source": traffic_source()}}
    if not args.no_cpu:
        import oracle
        n = 1 << 22
        rng = np.random.default_rng(0)
        p = rng.random(n).astype(np.float32); gr = rng.standard_normal(n).astype(np.float32)
        oracle.adam_steps(p, [gr])
        t = time.perf_counter(); reps = 20
        oracle.adam_steps(p, [gr] * reps)
        out["cpu_baseline"] = {"value": n * reps / (time.perf_counter() - t) / 1e9, "unit": "G updates/s", "cores": 1, "kind": "port",
                               "sample": "C restatement of the reference's host update, one tensor of %d elements, %d steps" % (n, reps)}
    return out


def library_timed_ms(lib, fn, steps, warmup, which=4):
    """Mean duration (ms) of the kernels one call of fn launches, from the HIP events that the library records around
    them on the launch stream (kind 4: the entries outside the LUT layers).  Events recorded by the caller would span
    the Python call as well, which is longer than these kernels."""
    import ctypes as C
    import torch
    from binarybrain_amd import capi
    for _ in range(warmup):
        out = fn(); del out
    torch.cuda.synchronize()
    lib.bbhip_KernelTimer_Enable(1)
    for _ in range(steps):
        out = fn(); del out
    torch.cuda.synchronize()
    lib.bbhip_KernelTimer_Enable(0)
    ms = C.c_float(0); cnt = C.c_int(0)
    capi.check(lib.bbhip_KernelTimer_Read(which, C.byref(ms), C.byref(cnt)))
    assert cnt.value == steps, (cnt.value, steps)
    return ms.value / cnt.value


def bench_conv(args, lib):
    """The permutation kernels around the LUT layers of a conv block (secondary measurement), at the shapes of the
    CIFAR-like configuration: 256 images of 3 x 32 x 32, 3 x 3 valid filter (27 taps, 230400 window frames), 36 output
    channels of 30 x 30, 2 x 2 pooling.  Algorithmic bytes: every element of input and output once."""
    import torch
    from binarybrain_amd import ops, synth
    F, C, H, W, FH, FW, CO = 256, 3, 32, 32, 3, 3, 36
    OH, OW = H - FH + 1, W - FW + 1
    g = torch.Generator(device="cuda"); g.manual_seed(0)
    img = torch.rand((C * H * W, synth.frame_stride_fp32(F)), device="cuda", generator=g)
    cols = ops.im2col_forward(img, C, H, W, F, FH, FW)
    dcols = torch.rand_like(cols)
    act = torch.rand((CO, synth.frame_stride_fp32(F * OH * OW)), device="cuda", generator=g)
    maps = ops.col2im_forward(act, CO, OH, OW, F)
    dmaps = torch.rand_like(maps)
    pooled = ops.stochastic_maxpool2x2_forward(maps, CO, OH, OW, F)
    dpooled = torch.rand_like(pooled)
    e = 4
    cases = [
        ("im2col_forward_kernel", lambda: ops.im2col_forward(img, C, H, W, F, FH, FW), e * F * (C * H * W + C * FH * FW * OH * OW)),
        ("im2col_backward_kernel", lambda: ops.im2col_backward(dcols, C, H, W, F, FH, FW), e * F * (C * H * W + C * FH * FW * OH * OW)),
        ("col2im_kernel<forward>", lambda: ops.col2im_forward(act, CO, OH, OW, F), 2 * e * F * CO * OH * OW),
        ("col2im_kernel<backward>", lambda: ops.col2im_backward(dmaps, CO, OH, OW, F), 2 * e * F * CO * OH * OW),
        ("stochastic_maxpool2x2_forward_kernel", lambda: ops.stochastic_maxpool2x2_forward(maps, CO, OH, OW, F), e * F * CO * (OH * OW + (OH // 2) * (OW // 2))),
        ("stochastic_maxpool2x2_backward_kernel", lambda: ops.stochastic_maxpool2x2_backward(maps, dpooled, CO, OH, OW, F),
         e * F * CO * (2 * OH * OW + (OH // 2) * (OW // 2))),
    ]
    kernels = {}
    total_ms = 0.0
    for name, fn, nbytes in cases:
        med = library_timed_ms(lib, fn, args.steps, args.warmup)
        total_ms += med
        kernels[name] = {"ms": med, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (med * 1e-3) / 1e9}
    dom = max(kernels, key=lambda k: kernels[k]["ms"])
    # MaxPooling (what binary networks pool with), UpSampling and Shuffle at the same maps, listed beside the block's own kernels, not added
    _, arg = ops.max_pooling_forward(maps, CO, OH, OW, 2, 2, F)
    PO = CO * (OH // 2) * (OW // 2)
    maps_bits = ops.binarize_forward(maps, F, 0.5, bit=True, y_stride=synth.frame_stride_bit(F))
    dup = torch.rand_like(maps)
    beside = [
        ("max_pooling_forward_kernel 2x2", lambda: ops.max_pooling_forward(maps, CO, OH, OW, 2, 2, F), e * F * (CO * OH * OW + 2 * PO)),
        ("max_pooling_backward_kernel 2x2", lambda: ops.max_pooling_backward(arg, dpooled, CO, OH, OW, 2, 2, F), e * F * (CO * OH * OW + 2 * PO)),
        ("max_pooling_bit_forward_kernel 2x2", lambda: ops.bit_max_pooling_forward(maps_bits, CO, OH, OW, 2, 2, F), F // 8 * (CO * OH * OW + PO)),
        ("max_pooling_bit_backward_kernel 2x2", lambda: ops.bit_max_pooling_backward(maps_bits, dpooled, CO, OH, OW, 2, 2, F),
         F // 8 * CO * OH * OW + e * F * (CO * OH * OW + PO)),
        ("up_sampling_forward_kernel 2x2", lambda: ops.up_sampling_forward(pooled, CO, OH // 2, OW // 2, 2, 2, F), e * F * (CO * OH * OW + PO)),
        ("up_sampling_backward_kernel 2x2", lambda: ops.up_sampling_backward(dup, CO, OH // 2, OW // 2, 2, 2, F), e * F * (CO * OH * OW + PO)),
        ("row_shuffle_kernel unit 36", lambda: ops.shuffle_forward(maps, CO, F), 2 * e * F * CO * OH * OW),
        ("row_shuffle_kernel unit 36, packed", lambda: ops.shuffle_forward(maps_bits, CO, F), 2 * 4 * maps_bits.shape[1] * CO * OH * OW),    # rows move whole
    ]
    for name, fn, nbytes in beside:
        med = library_timed_ms(lib, fn, args.steps, args.warmup)
        kernels[name] = {"ms": med, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (med * 1e-3) / 1e9}
    out = {"metric": "conv-block permutation kernels, ms per pass over 256 images (fwd+bwd)", "value": total_ms, "unit": "ms",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": total_ms, "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "Im2Col 3x32x32 (3x3 valid) / Col2Im 36x30x30 / StochasticMaxPooling2x2, 256 images"},
           "roofline": {"bound": "hbm", "kernel": dom, "achieved": kernels[dom]["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": kernels[dom]["achieved_GBps"] / HBM_PEAK_GBS, "traffic": None},
           "kernels": kernels}
    return out


def bench_stochastic_bn(args, lib):
    """StochasticBatchNormalization (secondary measurement) at the size of a hidden layer of the headline configuration, 8192 nodes
    x 4096 frames, and at the normalisation after a convolution, 32 channels x 50176 frames (few long rows: one workgroup per
    row).  Algorithmic bytes: every element of each input and output once (training and inference 8 B, backward 12 B per element)."""
    import torch
    from binarybrain_amd import ops, synth
    kernels = {}
    totals = {}
    for (nodes, F) in ((8192, 4096), (32, 50176)):
        g = torch.Generator(device="cuda"); g.manual_seed(0)
        S = synth.frame_stride_fp32(F)
        x = torch.rand((nodes, S), device="cuda", generator=g)
        dy = torch.randn((nodes, S), device="cuda", generator=g)
        rm = torch.zeros(nodes, device="cuda"); rv = torch.ones(nodes, device="cuda")
        _, mean, rstd = ops.stochastic_bn_forward_training(x, rm, rv, F)
        e = 4 * nodes * F
        cases = [
            ("bn_forward_training_kernel", lambda: ops.stochastic_bn_forward_training(x, rm, rv, F), 2 * e),
            ("bn_backward_kernel", lambda: ops.stochastic_bn_backward(x, dy, mean, rstd, F), 3 * e),
            ("bn_apply_kernel (inference)", lambda: ops.stochastic_bn_forward_inference(x, rm, rv, F), 2 * e),
        ]
        total_ms = 0.0
        for name, fn, nbytes in cases:
            med = library_timed_ms(lib, fn, args.steps, args.warmup)
            total_ms += med
            kernels["%s %dx%d" % (name, nodes, F)] = {"ms": med, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (med * 1e-3) / 1e9}
        totals[(nodes, F)] = total_ms
    big = {k: v for k, v in kernels.items() if k.endswith("8192x4096")}
    dom = max(big, key=lambda k: big[k]["ms"])
    ms = totals[(8192, 4096)]
    out = {"metric": "StochasticBatchNormalization training fwd + bwd + inference, ms per pass over 8192 nodes x 4096 frames", "value": ms,
           "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "StochasticBatchNormalization fp32, 8192 nodes x 4096 frames", "ms_at_32x50176": totals[(32, 50176)]},
           "roofline": {"bound": "hbm", "kernel": dom, "achieved": big[dom]["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": big[dom]["achieved_GBps"] / HBM_PEAK_GBS, "traffic": None},
           "kernels": kernels}
    return out


def bench_modulation(args, lib):
    """RealToBinary, BinaryToReal, Binarize and HardTanh (secondary measurement).  The converters at the size of an MNIST-like input
    batch (784 nodes x 4096 frames, 7 frames per input: 28672 modulated frames) and of a classifier's last binary layer (1024 nodes
    folding into 128, 7 frames into 1); the activations at the size of a hidden layer of the headline configuration, 8192 nodes x
    4096 frames.  Algorithmic bytes: every element of each input and output once (4 B per fp32 element, 1 bit per packed one)."""
    import torch
    from binarybrain_amd import ops, synth
    g = torch.Generator(device="cuda"); g.manual_seed(0)
    nodes, F, fm = 784, 4096, 7
    yF = F * fm
    x = torch.rand((nodes, synth.frame_stride_fp32(F)), device="cuda", generator=g)
    ys, ws = synth.frame_stride_fp32(yF), synth.frame_stride_bit(yF)
    I, O = 1024, 128
    h = (torch.rand((I, ys), device="cuda", generator=g) - 0.5)
    hb = ops.binarize_forward(h, yF, 0.0, bit=True, y_stride=ws)
    dyo = torch.randn((O, synth.frame_stride_fp32(F)), device="cuda", generator=g)
    an, aF = 8192, 4096
    aS = synth.frame_stride_fp32(aF)
    a = torch.randn((an, aS), device="cuda", generator=g)
    da = torch.randn((an, aS), device="cuda", generator=g)
    e = 4
    cases = [
        ("real_to_binary_kernel fp32 784x4096 x7", lambda: ops.real_to_binary_forward(x, 1, nodes, F, fm, y_stride=ys), e * nodes * (F + yF)),
        ("real_to_binary_kernel bit 784x4096 x7", lambda: ops.real_to_binary_forward(x, 1, nodes, F, fm, bit=True, y_stride=ws), e * nodes * F + nodes * yF // 8),
        ("binary_to_real_forward_kernel fp32 1024->128 /7", lambda: ops.binary_to_real_forward(h, O, F, fm), e * (I * yF + O * F)),
        ("binary_to_real_forward_kernel bit 1024->128 /7", lambda: ops.binary_to_real_forward(hb, O, F, fm), I * yF // 8 + e * O * F),
        ("binary_to_real_backward_kernel 128->1024 x7", lambda: ops.binary_to_real_backward(dyo, I, F, fm, x_stride=ys), e * (O * F + I * yF)),
        ("row_map_kernel Binarize 8192x4096", lambda: ops.binarize_forward(a, aF), 2 * e * an * aF),
        ("binarize_bits_kernel 8192x4096", lambda: ops.binarize_forward(a, aF, bit=True, y_stride=synth.frame_stride_bit(aF)), e * an * aF + an * aF // 8),
        ("row_map_kernel HardTanh 8192x4096", lambda: ops.hard_tanh_forward(a, aF), 2 * e * an * aF),
        ("row_map_kernel HardTanh backward 8192x4096", lambda: ops.hard_tanh_backward(a, da, aF), 3 * e * an * aF),
    ]
    kernels = {}
    total_ms = 0.0
    for name, fn, nbytes in cases:
        med = library_timed_ms(lib, fn, args.steps, args.warmup)
        total_ms += med
        kernels[name] = {"ms": med, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (med * 1e-3) / 1e9}
    dom = max(kernels, key=lambda k: kernels[k]["ms"])
    out = {"metric": "RealToBinary + BinaryToReal + Binarize + HardTanh kernels, ms for one launch of each", "value": total_ms, "unit": "ms",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": total_ms, "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "converters at 784 nodes x 4096 frames x 7 and 1024 -> 128 nodes; activations at 8192 nodes x 4096 frames"},
           "roofline": {"bound": "hbm", "kernel": dom, "achieved": kernels[dom]["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": kernels[dom]["achieved_GBps"] / HBM_PEAK_GBS, "traffic": None},
           "kernels": kernels}
    return out


def bench_tail(args, lib):
    """The tail of the MNIST-like classifier (secondary measurement): AverageLut 7 -> 1 over 70 -> 10 nodes (and MaxLut at the same
    shape), softmax cross entropy and categorical accuracy over the 10 classes.  Measured at 65536 frames (streaming rate) and at the
    configuration's own batch of 1024 frames (launch-bound).  Algorithmic bytes: every element of input and output once."""
    import numpy as np
    import torch
    from binarybrain_amd import ops, synth
    n, I, O = 7, 70, 10
    kernels = {}
    totals = {}
    fused = {}
    for F in (65536, 1024):
        g = torch.Generator(device="cuda"); g.manual_seed(0)
        S = synth.frame_stride_fp32(F)
        idx = torch.arange(I, dtype=torch.int32, device="cuda").reshape(O, n).contiguous()
        x = torch.rand((I, S), device="cuda", generator=g)
        dy = torch.rand((O, S), device="cuda", generator=g)
        y = torch.rand((O, S), device="cuda", generator=g)
        t = torch.zeros((O, S), device="cuda")
        label = torch.randint(0, O, (F,), device="cuda", generator=g)
        t[label, torch.arange(F, device="cuda")] = 1.0
        e = 4
        cases = [
            ("average_lut_forward_kernel", lambda: ops.average_lut_forward(x, idx, F, False, False), e * F * (I + O)),
            ("average_lut_backward_kernel (+ reverse wiring)", lambda: ops.average_lut_backward(dy, idx, I, F), e * F * (I + O)),
            ("max_lut_forward_kernel", lambda: ops.max_lut_forward(x, idx, F, False, False), e * F * (I + O)),
            ("max_lut_backward_kernel (+ reverse wiring)", lambda: ops.max_lut_backward(x, dy, idx, F), e * F * (2 * I + O)),
            ("softmax_cross_entropy_kernel", lambda: ops.loss_softmax_cross_entropy(y, t, O, 1, F, t_sum=float(F)), e * F * 3 * O + 8 * F),
            ("categorical_accuracy_kernel", lambda: ops.metrics_categorical_accuracy(y, t, O, 1, F), e * F * 2 * O + 8 * F),
        ]
        total_ms = 0.0
        for name, fn, nbytes in cases:
            med = library_timed_ms(lib, fn, args.steps, args.warmup)
            if not name.startswith("max_lut"):          # the classifier's tail uses AverageLut; MaxLut is listed beside it, not added
                total_ms += med
            if F == 65536:
                kernels[name] = {"ms": med, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (med * 1e-3) / 1e9}
        totals[F] = total_ms
        # the same four (AverageLut forward, loss, accuracy, AverageLut backward) as the one launch of bbhip_fp32_ClassifierTail_ForwardBackward
        fused[F] = library_timed_ms(lib, lambda: ops.classifier_tail(x, idx, t, F, t_sum=float(F)), args.steps, args.warmup)
    dom = max((k for k in kernels if not k.startswith("max_lut")), key=lambda k: kernels[k]["ms"])
    out = {"metric": "classifier tail (AverageLut fwd+bwd, softmax cross entropy, accuracy), ms per pass over 65536 frames", "value": totals[65536],
           "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": totals[65536], "higher_is_better": False,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "AverageLut 7->1 over 70->10 nodes + LossSoftmaxCrossEntropy + MetricsCategoricalAccuracy, 65536 frames (MaxLut at the same shape listed under kernels)",
                      "ms_at_1024_frames": totals[1024], "ms_as_one_launch": fused[65536], "ms_as_one_launch_at_1024_frames": fused[1024]},
           "roofline": {"bound": "hbm", "kernel": dom, "achieved": kernels[dom]["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": kernels[dom]["achieved_GBps"] / HBM_PEAK_GBS, "traffic": None},
           "kernels": kernels}
    return out


def bench_differentiablelut6(args, lib):
    """DifferentiableLut6 training step (secondary measurement): the LUT fused with per-node batch normalisation in binary
    mode (the class defaults), forward (statistics pass, normalising pass) and backward (statistics pass, table-gradient
    pass, input-centric dx) at the shape of the headline workload."""
    import numpy as np
    import torch
    from binarybrain_amd import ops, synth
    I = O = 4096
    F = 8192
    rng = np.random.default_rng(0)
    idx = torch.from_numpy(synth.wiring(rng, I, O)).cuda()
    W = torch.from_numpy(synth.lut_tables(rng, O)).cuda()
    S = synth.frame_stride_fp32(F)
    x = torch.from_numpy(synth.uniform_frames(rng, I, F, S)).cuda()
    dy = torch.from_numpy(synth.normal_frames(rng, O, F, S)).cuda()
    dW = torch.zeros((O, 64), device="cuda")
    rm = torch.zeros(O, device="cuda"); rv = torch.ones(O, device="cuda")
    ops.set_dx_mode(0)
    rev = ops.reverse_table(idx, I)
    bits = args.workload.endswith("_bit")
    if bits:
        xb = torch.from_numpy(synth.bernoulli_bits(rng, I, F, synth.frame_stride_bit(F))).cuda()

    tables = ops.prepared_tables_buffer(6, idx.shape[0])     # the model class keeps the tables derived from W from forward to backward
    packed = ops.packed_input_buffer(I, F)                   # ... and the packed copy of its binarized input
    plain = getattr(args, "plain_signatures", False)
    clamp_w = None if plain else (0.0, 1.0)
    yb = torch.zeros((idx.shape[0], xb.shape[1]), dtype=torch.int32, device="cuda") if bits else None      # the layer's packed output buffer

    def step():
        # (the table is clamped to [0, 1] in place by the forward entry, as the model class does before a forward pass; with the
        # reference's plain signatures the clamp is a launch of its own)
        if plain:
            ops.vector_clamp_(W, 0.0, 1.0)
        if bits:
            y, mean, rstd = ops.bit_differentiable_lut_forward_training(6, xb, idx, W, F, rm, rv, clamp_w=clamp_w, tables=tables, out=yb)
            ops.bit_differentiable_lut_backward(6, xb, dy, idx, W, dW, F, mean, rstd, rev, tables=tables)
        else:
            y, mean, rstd = ops.differentiable_lut_forward_training(6, x, idx, W, F, rm, rv, clamp_w=clamp_w, packed=packed, tables=tables)
            ops.differentiable_lut_backward(6, x, dy, idx, W, dW, F, mean, rstd, rev, packed=packed, tables=tables)

    ops.HINTS = not plain
    try:
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < args.ramp_seconds:
            for _ in range(10):
                step()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    finally:
        ops.HINTS = True
    # every tensor once per pass: forward x, y, tables; backward x, dy, dx, tables, per-node statistics
    nbytes = 4 * F * (I + O) + 4 * F * (2 * I + O) + 4 * 280 * O + 32 * O
    if bits:      # packed x and y (1 bit per element), fp32 dy and dx
        nbytes = (F // 8) * (I + O) + (F // 8) * I + 4 * F * (I + O) + 4 * 280 * O + 32 * O
    out = {"metric": "G node-evals/s DifferentiableLut6 %s fwd+bwd with batch-norm, binary mode (8192 frames x 4096 nodes)" % ("packed-bit" if bits else "fp32"),
           "value": O * F / dt / 1e9, "unit": "G node-evals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "DifferentiableLut6 training fwd+bwd %s (batch_norm, binary), 4096 in x 4096 out x 8192 frames"
                                  % ("packed-bit activations, fp32 gradients" if bits else "fp32")},
           "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "traffic": None}}
    return out


def conv_block_layers(rng, synth, ops, torch, np):
    """wiring and tables of the two per-pixel LUT layers of the conv block (27 -> 216 -> 36)"""
    layers = []
    for I, O in ((27, 216), (216, 36)):
        idx = torch.from_numpy(synth.wiring(rng, I, O)).cuda()
        W = torch.from_numpy((0.5 + 0.1 * rng.standard_normal((O, 64))).astype(np.float32)).cuda()
        layers.append(dict(I=I, O=O, idx=idx, W=W, dW=torch.zeros_like(W), rm=torch.zeros(O, device="cuda"), rv=torch.ones(O, device="cuda"),
                           rev=ops.reverse_table(idx, I)))
    return layers


def bench_conv_block(args, lib):
    """Forward + backward of the convolutional LUT block (secondary measurement): 256 images of 3 x 32 x 32, Im2Col 3 x 3 valid
    (27 taps, 230400 window frames), DifferentiableLut6 27 -> 216 -> 36 per pixel with batch-norm in binary mode, Col2Im to
    36 x 30 x 30, StochasticMaxPooling2x2 to 36 x 15 x 15, and the backward pass of all of it down to the image gradient."""
    import numpy as np
    import torch
    from binarybrain_amd import ops, synth
    F, C, H, W_, FH, FW, CO = 256, 3, 32, 32, 3, 3, 36
    OH, OW = H - FH + 1, W_ - FW + 1
    FW_FRAMES = F * OH * OW
    rng = np.random.default_rng(0)
    layers = conv_block_layers(rng, synth, ops, torch, np)
    g = torch.Generator(device="cuda"); g.manual_seed(0)
    img = torch.rand((C * H * W_, synth.frame_stride_fp32(F)), device="cuda", generator=g)
    dpooled = torch.randn((CO * (OH // 2) * (OW // 2), synth.frame_stride_fp32(F)), device="cuda", generator=g)
    ops.set_dx_mode(0)

    # what a caller that keeps a layer's input for the backward pass keeps as well (the model classes do): the packed copy of each
    # layer's binarized input — the first layer's is packed by its forward call, the second layer's is written by the first layer's
    # forward call as its packed output — and the tables derived from W
    for l in layers:
        l["packed_in"] = ops.packed_input_buffer(l["I"], FW_FRAMES)
        l["tables"] = ops.prepared_tables_buffer(6, l["O"])

    plain = getattr(args, "plain_signatures", False)
    clamp_w = None if plain else (0.0, 1.0)

    def step():
        cols = ops.im2col_forward(img, C, H, W_, F, FH, FW)
        a = cols; acts = []
        for k, l in enumerate(layers):
            # the model class clamps its table before the first forward pass after a backward pass; the entry does it with its tables
            # (with the reference's plain signatures the clamp is a launch of its own)
            if plain:
                ops.vector_clamp_(l["W"], 0.0, 1.0)
            nxt = layers[k + 1]["packed_in"] if k + 1 < len(layers) else None
            y, mean, rstd = ops.differentiable_lut_forward_training(6, a, l["idx"], l["W"], FW_FRAMES, l["rm"], l["rv"], clamp_w=clamp_w,
                                                                    packed=l["packed_in"], packed_holds=(k > 0), packed_out=nxt, tables=l["tables"])
            acts.append((a, mean, rstd)); a = y
        maps = ops.col2im_forward(a, CO, OH, OW, F)
        pooled = ops.stochastic_maxpool2x2_forward(maps, CO, OH, OW, F)
        dmaps = ops.stochastic_maxpool2x2_backward(maps, dpooled, CO, OH, OW, F)
        dy = ops.col2im_backward(dmaps, CO, OH, OW, F)
        for l, (a_in, mean, rstd) in zip(reversed(layers), reversed(acts)):
            # one backward pass per step and no optimizer in it: the table gradient is written, not accumulated (a fill launch otherwise)
            if not ops.HINTS:
                l["dW"].zero_()
            dy = ops.differentiable_lut_backward(6, a_in, dy, l["idx"], l["W"], l["dW"], FW_FRAMES, mean, rstd, l["rev"], packed=l["packed_in"],
                                                 tables=l["tables"], overwrite_dw=ops.HINTS)
        return ops.im2col_backward(dy, C, H, W_, F, FH, FW), pooled

    ops.HINTS = not plain
    try:
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < args.ramp_seconds:
            for _ in range(3):
                step()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    finally:
        ops.HINTS = True
    node_evals = sum(l["O"] for l in layers) * FW_FRAMES
    e = 4
    # every activation and gradient once per pass: image, window columns, both LUT layers, maps, pooled maps
    nbytes = (e * F * (C * H * W_ + 27 * OH * OW) * 2 + sum(e * FW_FRAMES * (3 * l["I"] + 2 * l["O"]) for l in layers)
              + 2 * e * F * CO * OH * OW * 2 + e * F * CO * (OH * OW * 3 + 2 * (OH // 2) * (OW // 2)))
    out = {"metric": "G node-evals/s, convolutional DifferentiableLut6 block 27->216->36 per pixel, 256 images of 3x32x32, fwd+bwd",
           "value": node_evals / dt / 1e9, "unit": "G node-evals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "Im2Col 3x3 -> DifferentiableLut6 27->216->36 (batch_norm, binary) -> Col2Im 36x30x30 -> StochasticMaxPooling2x2, "
                                  "256 images of 3x32x32, forward + backward", "images_per_s": F / dt},
           "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "traffic": None if plain else measured_traffic("steps", "conv_block"),
                        "traffic_source": traffic_source()}}
    if not args.no_cpu:
        import oracle
        Fs = 4                                                # images in the CPU sample
        S = synth.frame_stride_fp32(Fs); FWs = Fs * OH * OW
        xs = np.zeros((C * H * W_, S), np.float32); xs[:, :Fs] = img[:, :Fs].cpu().numpy()
        Ws = [l["W"].cpu().numpy() for l in layers]; idxs = [l["idx"].cpu().numpy() for l in layers]
        dps = np.ascontiguousarray(dpooled[:, :Fs].cpu().numpy())          # the oracle's conv functions work on dense rows
        threads = min(os.cpu_count() or 1, 16)
        if oracle.have_ref():
            # the reference's own classes (oracle/_ref: its headers compiled in place; OpenMP forward, single-threaded batch-norm backward).
            # Untimed: one forward pass for the activations.  Timed: every layer's Forward + Backward, last layer first.
            os.environ.setdefault("OMP_NUM_THREADS", str(threads))
            dense = lambda a_, n_: np.ascontiguousarray(a_[:, :n_])
            cols, _ = oracle.ref_im2col(dense(xs, Fs), C, H, W_, Fs, FH, FW)
            a = cols; ins = []
            for l, Wt, idx in zip(layers, Ws, idxs):
                ins.append(a)
                a = oracle.ref_differentiable_lut(6, a, idx, Wt, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32))["y"]
            maps, _ = oracle.ref_col2im(a, CO, OH, OW, Fs)
            t0 = time.perf_counter()
            oracle.ref_im2col(dense(xs, Fs), C, H, W_, Fs, FH, FW)
            _, dmaps = oracle.ref_stochastic_maxpool2x2(maps, CO, OH, OW, Fs, dy=dps)
            _, dy = oracle.ref_col2im(a, CO, OH, OW, Fs, dy=dmaps)
            for l, Wt, idx, a_in in zip(reversed(layers), reversed(Ws), reversed(idxs), reversed(ins)):
                dy = oracle.ref_differentiable_lut(6, a_in, idx, Wt, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32), dy=dy)["dx"]
            oracle.ref_im2col(dense(xs, Fs), C, H, W_, Fs, FH, FW, dy=dy)
            cpu_dt = time.perf_counter() - t0
            out["cpu_baseline"] = {"value": sum(l["O"] for l in layers) * FWs / cpu_dt / 1e9, "unit": "G node-evals/s", "cores": threads, "kind": "reference",
                                   "sample": "the same block on %d of the 256 images through the reference's own host classes (Forward + Backward of every layer incl. the "
                                             "harness's buffer copies; its DifferentiableLut forward runs on the OpenMP threads, its batch-norm backward on one)" % Fs}
        else:
            t0 = time.perf_counter()
            a = oracle.im2col_forward(xs, C, H, W_, Fs, FH, FW); acts = []
            for l, Wt, idx in zip(layers, Ws, idxs):
                y, mean, rstd, _, _ = oracle.differentiable_lut_forward_training(6, a, idx, Wt, FWs, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32))
                acts.append((a, mean, rstd)); a = y
            maps = oracle.col2im_forward(a, CO, OH, OW, Fs)
            oracle.stochastic_maxpool2x2_forward(maps, CO, OH, OW, Fs)
            dy = oracle.col2im_backward(oracle.stochastic_maxpool2x2_backward(maps, dps, CO, OH, OW, Fs), CO, OH, OW, Fs)
            for l, Wt, idx, (a_in, mean, rstd) in zip(reversed(layers), reversed(Ws), reversed(idxs), reversed(acts)):
                dy, _ = oracle.differentiable_lut_backward(6, a_in, dy, idx, Wt, FWs, mean, rstd)
            oracle.im2col_backward(dy, C, H, W_, Fs, FH, FW)
            cpu_dt = time.perf_counter() - t0
            out["cpu_baseline"] = {"value": sum(l["O"] for l in layers) * FWs / cpu_dt / 1e9, "unit": "G node-evals/s", "cores": 1, "kind": "port",
                                   "sample": "the same block on %d images through the C restatement of the reference's host path (generic DifferentiableLut "
                                             "algorithm, whose batch-norm backward is single-threaded in the reference too)" % Fs}
    return out


def bench_mnist_step(args, lib):
    """One training step of the MNIST-like LUT classifier (secondary measurement; launch- and latency-bound): DifferentiableLut6
    784 -> 6144 -> 1024 -> 70 with batch-norm in binary mode, AverageLut 7 -> 1 (10 classes), softmax cross entropy,
    accuracy, Adam, 1024 frames.  Timed twice: every entry point called from the host per step, and the forward + backward
    part of the step replayed as one HIP graph (captured from the same calls on a torch capture stream; Adam stays a
    launch of its own because its bias-corrected rate is a host scalar that changes per step)."""
    import numpy as np
    import torch
    from binarybrain_amd import ops, synth
    sizes = [784, 6144, 1024, 70]
    CLASSES, N_AVG, F = 10, 7, 1024
    rng = np.random.default_rng(0)
    S = synth.frame_stride_fp32(F)
    layers = []
    for I, O in zip(sizes[:-1], sizes[1:]):
        idx = torch.from_numpy(synth.wiring(rng, I, O)).cuda()
        W = torch.from_numpy((0.5 + 0.01 * rng.standard_normal((O, 64))).astype(np.float32)).cuda()
        layers.append(dict(I=I, O=O, idx=idx, W=W, dW=torch.zeros_like(W), rm=torch.zeros(O, device="cuda"), rv=torch.ones(O, device="cuda"),
                           rev=ops.reverse_table(idx, I)))
    idx_avg = torch.arange(sizes[-1], dtype=torch.int32, device="cuda").reshape(CLASSES, N_AVG).contiguous()
    x = torch.from_numpy(synth.uniform_frames(rng, sizes[0], F, S)).cuda()
    t = torch.zeros((CLASSES, S), device="cuda")
    label = torch.from_numpy(rng.integers(0, CLASSES, F)).cuda()
    t[label, torch.arange(F, device="cuda")] = 1.0
    adam = ops.AdamState([l["W"] for l in layers], [l["dW"] for l in layers], learning_rate=0.001)
    ops.set_dx_mode(0)
    keep = {}

    # what a caller that keeps a layer's input for the backward pass keeps as well (the model classes do): the packed copy of each
    # layer's binarized input — the first layer's is packed by its forward call, every other layer's is written by the forward call of
    # the layer before as its packed output — and the tables derived from W
    for l in layers:
        l["packed_in"] = ops.packed_input_buffer(l["I"], F)
        l["tables"] = ops.prepared_tables_buffer(6, l["O"])

    plain = getattr(args, "plain_signatures", False)
    clamp_w = None if plain else (0.0, 1.0)

    def forward_backward():
        a = x
        acts = []
        for k, l in enumerate(layers):
            # the model class clamps its table before the first forward pass after a backward pass; the entry does it with its tables
            # (with the reference's plain signatures the clamp is a launch of its own)
            if plain:
                ops.vector_clamp_(l["W"], 0.0, 1.0)
            nxt = layers[k + 1]["packed_in"] if k + 1 < len(layers) else None
            y, mean, rstd = ops.differentiable_lut_forward_training(6, a, l["idx"], l["W"], F, l["rm"], l["rv"], clamp_w=clamp_w,
                                                                    packed=l["packed_in"], packed_holds=(k > 0), packed_out=nxt, tables=l["tables"])
            acts.append((a, mean, rstd)); a = y
        if plain:
            out = ops.average_lut_forward(a, idx_avg, F, False, False, mean=False)
            dy, loss_buf, _ = ops.loss_softmax_cross_entropy(out, t, CLASSES, 1, F, t_sum=float(F))
            acc, cat = ops.metrics_categorical_accuracy(out, t, CLASSES, 1, F)
            dy = ops.average_lut_backward(dy, idx_avg, sizes[-1], F)
        else:       # the same four in one launch
            out, dy, loss_buf, acc, cat, _ = ops.classifier_tail(a, idx_avg, t, F, t_sum=float(F), mean=False)
        for l, (a_in, mean, rstd) in zip(reversed(layers), reversed(acts)):
            # dW accumulates; it is zero here because the optimizer's Update() zeroed it after the previous step (Optimizer.h:31-35)
            dy = ops.differentiable_lut_backward(6, a_in, dy, l["idx"], l["W"], l["dW"], F, mean, rstd, l["rev"], packed=l["packed_in"], tables=l["tables"])
        keep["loss_buf"], keep["acc"] = loss_buf, acc

    def timed(fn):
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < args.ramp_seconds:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    def optimizer_update():
        if plain:               # bbcu_fp32_OptimizerAdam, then the gradients cleared tensor by tensor (Optimizer::Update, include/bb/Optimizer.h:31-35)
            adam.step()
            for l in layers:
                ops.vector_set_(l["dW"], 0.0)
        else:
            adam.update()

    def eager_step():
        forward_backward(); optimizer_update()

    ops.HINTS = not plain
    try:
        dt_eager = timed(eager_step)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            forward_backward()

        def graph_step():
            graph.replay(); optimizer_update()

        dt_graph = timed(graph_step)
    finally:
        ops.HINTS = True
    loss = -float(keep["loss_buf"].sum().item()) / F
    node_evals = sum(sizes[1:]) * F
    # every activation, gradient and table once per pass over the three LUT layers
    nbytes = sum(4 * F * (3 * l["I"] + 2 * l["O"]) + 4 * 280 * l["O"] * 2 for l in layers)
    dt = min(dt_eager, dt_graph)
    out = {"metric": "training steps/s, MNIST-like DifferentiableLut6 classifier 784-6144-1024-70, 1024 frames", "value": 1.0 / dt,
           "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "DifferentiableLut6 784->6144->1024->70 (batch_norm, binary) + AverageLut 7->1 + softmax CE + accuracy + Adam, 1024 frames",
                      "ms_per_step_host_launched": dt_eager * 1e3, "ms_per_step_graph_replay": dt_graph * 1e3,
                      "G_node_evals_per_s": node_evals / dt / 1e9, "loss_after_run": loss},
           "roofline": {"bound": "hbm", "kernel": "whole step (launch-bound)", "achieved": nbytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / dt / 1e9 / HBM_PEAK_GBS, "traffic": None if plain else measured_traffic("steps", "mnist_step"),
                        "traffic_source": traffic_source()}}
    if not args.no_cpu:
        import oracle
        xs = x.cpu().numpy(); ts = t.cpu().numpy()
        Ws = [l["W"].cpu().numpy() for l in layers]; idxs = [l["idx"].cpu().numpy() for l in layers]
        threads = min(os.cpu_count() or 1, 16)
        if oracle.have_ref():
            # the reference's own classes (oracle/_ref).  Untimed: one forward pass for the activations.  Timed: the tail, then every
            # layer's Forward + Backward, last layer first, each fed the gradient that the layer behind it returned.
            os.environ.setdefault("OMP_NUM_THREADS", str(threads))
            a = np.ascontiguousarray(xs[:, :F]); ins = []
            for l, W, idx in zip(layers, Ws, idxs):
                ins.append(a)
                a = oracle.ref_differentiable_lut(6, a, idx, W, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32))["y"]
            t0 = time.perf_counter()
            o = oracle.average_lut_forward(a, idx_avg.cpu().numpy(), F, False, False)
            dy, _, _ = oracle.loss_softmax_cross_entropy(o, np.ascontiguousarray(ts[:, :F]), CLASSES, 1, F)
            dy = oracle.average_lut_backward(dy, idx_avg.cpu().numpy(), sizes[-1], F)
            for l, W, idx, a_in in zip(reversed(layers), reversed(Ws), reversed(idxs), reversed(ins)):
                dy = oracle.ref_differentiable_lut(6, a_in, idx, W, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32), dy=dy)["dx"]
            cpu_dt = time.perf_counter() - t0
            out["cpu_baseline"] = {"value": 1.0 / cpu_dt, "unit": "steps/s", "cores": threads, "kind": "reference",
                                   "sample": "Forward + Backward of the three DifferentiableLut6 layers through the reference's own host class (incl. the harness's "
                                             "buffer copies; its forward runs on the OpenMP threads, its batch-norm backward on one), the 70-node tail through "
                                             "the C restatement, Adam not included"}
        else:
            t0 = time.perf_counter()
            a = xs; acts = []
            for l, W, idx in zip(layers, Ws, idxs):
                y, mean, rstd, _, _ = oracle.differentiable_lut_forward_training(6, a, idx, W, F, np.zeros(l["O"], np.float32), np.ones(l["O"], np.float32))
                acts.append((a, mean, rstd)); a = y
            o = oracle.average_lut_forward(a, idx_avg.cpu().numpy(), F, False, False)
            dy, _, _ = oracle.loss_softmax_cross_entropy(o, ts, CLASSES, 1, F)
            dy = oracle.average_lut_backward(dy, idx_avg.cpu().numpy(), sizes[-1], F)
            for l, W, idx, (a_in, mean, rstd) in zip(reversed(layers), reversed(Ws), reversed(idxs), reversed(acts)):
                dy, _ = oracle.differentiable_lut_backward(6, a_in, dy, idx, W, F, mean, rstd)
            cpu_dt = time.perf_counter() - t0
            out["cpu_baseline"] = {"value": 1.0 / cpu_dt, "unit": "steps/s", "cores": 1, "kind": "port",
                                   "sample": "one forward + backward of the same network through the C restatement of the reference's generic "
                                             "DifferentiableLut path (its batch-norm backward is single-threaded in the reference too), Adam not included"}
    return out


def bench_binarylut6(args, lib):
    """BinaryLut6 packed inference: 8192 -> 16384 nodes, 262144 frames, 32 frames per word (secondary measurement)."""
    import numpy as np
    import torch
    from binarybrain_amd import capi, ops, synth
    I, O, F = 8192, 16384, 262144
    SW = synth.frame_stride_bit(F)
    rng = np.random.default_rng(0)
    idx = torch.from_numpy(synth.wiring(rng, I, O)).cuda()
    T = torch.from_numpy(synth.truth_tables(rng, O)).cuda()
    x = torch.from_numpy(synth.bernoulli_bits(rng, I, F, SW)).cuda()
    y = torch.zeros((O, SW), dtype=torch.int32, device="cuda")
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < args.ramp_seconds:      # untimed: the device reaches its sustained clock under load
        for _ in range(10):
            ops.binary_lut6_forward(x, idx, T, F, out=y)
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        ops.binary_lut6_forward(x, idx, T, F, out=y)
    torch.cuda.synchronize()
    lib.bbhip_KernelTimer_Enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ops.binary_lut6_forward(x, idx, T, F, out=y)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lib.bbhip_KernelTimer_Enable(0)
    ms = C.c_float(); cnt = C.c_int()
    capi.check(lib.bbhip_KernelTimer_Read(2, C.byref(ms), C.byref(cnt)))
    avg_ms = ms.value / max(cnt.value, 1)
    alg = F // 8 * (I + O) + 32 * O
    gbs = alg / (avg_ms * 1e-3) / 1e9
    out = {"metric": "T node-evals/s BinaryLut6 packed inference (8192 -> 16384 nodes, 262144 frames)",
           "value": O * F / (dt / args.steps) / 1e12, "unit": "T node-evals/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "u32", "data": "synthetic",
           "config": {"workload": "BinaryLut6 packed inference, 8192 in x 16384 out x 262144 frames", "frame_stride_words": SW},
           "roofline": {"bound": "hbm", "kernel": "binary_lut6_kernel", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": gbs / HBM_PEAK_GBS,
                        "traffic": measured_traffic("kernels", "binarylut6/binary_lut6_kernel"), "traffic_source": traffic_source()}}
    if args.profile_copy:
        for _ in range(3):
            y[:I].copy_(x)
        torch.cuda.synchronize()
        out["profile_copy_bytes"] = int(x.numel() * 4)
    if not args.no_cpu:
        import oracle
        os.environ.setdefault("OMP_NUM_THREADS", str(min(os.cpu_count() or 1, 16)))
        fs = 8192                                        # bounded sample: same nodes, 8192 of the 262144 frames
        xs = synth.bernoulli_bits(rng, I, fs)
        idx_h = idx.cpu().numpy(); T_h = T.cpu().numpy()
        best = None
        for _ in range(3):
            t1 = time.perf_counter()
            if oracle.have_ref():
                oracle.ref_binary_lut6(xs, idx_h, T_h, fs, host_simd=True)
            else:
                oracle.binary_lut6_forward(xs, idx_h, T_h, fs, words=True)
            d = time.perf_counter() - t1
            best = d if best is None else min(best, d)
        out["cpu_baseline"] = {"value": O * fs / best / 1e12, "unit": "T node-evals/s", "cores": min(os.cpu_count() or 1, 16),
                               "kind": "reference" if oracle.have_ref() else "port",
                               "sample": "BinaryLut6 forward (AVX2+OpenMP host path incl. harness copies), 8192 -> 16384 nodes, 8192 of the 262144 frames, best of 3"}
    return out


def bench_stochasticlut6(args, lib):
    """The headline workload: W clamp + StochasticLut6 forward + backward (dW, dx), fp32, 4096 -> 4096 nodes, 8192 frames."""
    import numpy as np
    import torch
    from binarybrain_amd import capi, ops, synth
    I = O = 4096
    F = 8192
    rng = np.random.default_rng(0)
    idx_h = synth.wiring(rng, I, O)
    idx = torch.from_numpy(idx_h).cuda()
    W = torch.from_numpy(synth.lut_tables(rng, O)).cuda()
    S = synth.frame_stride_fp32(F)                     # node rows padded off a power-of-two pitch
    x = torch.from_numpy(synth.uniform_frames(rng, I, F, S)).cuda()
    dy = torch.from_numpy(synth.normal_frames(rng, O, F, S)).cuda()
    dW = torch.zeros((O, 64), device="cuda")
    y = torch.empty((O, S), device="cuda")
    dx = torch.empty((I, S), device="cuda")
    ops.set_dx_mode(args.dx_mode)
    rev = ops.reverse_table(idx, I) if args.dx_mode != 1 else None
    dx_tmp = None
    tmp_frames = None
    if args.dx_mode == 2:
        tmp_frames = ops._tmp_frames(O, 6, F, args.tmp_mb << 20)
        dx_tmp = torch.empty((O * 6, ((tmp_frames + 63) // 64) * 64), device="cuda")

    def step():
        # StochasticLutN::Forward clamps W to [0, 1] in place first: the forward entry does that in its table-preparation launch
        if args.separate_clamp:
            ops.vector_clamp_(W)
            ops.stochastic_lut_forward(6, x, idx, W, F, out=y)
        else:
            ops.stochastic_lut_forward(6, x, idx, W, F, out=y, clamp_w=(0.0, 1.0))
        ops.stochastic_lut_backward(6, x, dy, idx, W, dW, F, rev, dx_tmp=dx_tmp, tmp_frame_size=tmp_frames, out=dx)

    t_ramp = time.perf_counter()
    ramp_steps = 0
    while time.perf_counter() - t_ramp < args.ramp_seconds:
        for _ in range(10):
            step()
        ramp_steps += 10
        torch.cuda.synchronize()
    ramp_done = time.perf_counter() - t_ramp
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly K steps, nothing else on the stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # the same K steps once more with the library's HIP events around the three main kernels (on the launch stream): the
    # event records cost about 3 us each on the device, so they stay out of the region that `value` is computed from
    lib.bbhip_KernelTimer_Enable(1)
    t1 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt_events = time.perf_counter() - t1
    lib.bbhip_KernelTimer_Enable(0)

    def read_timer(which):
        ms = C.c_float(); cnt = C.c_int()
        capi.check(lib.bbhip_KernelTimer_Read(which, C.byref(ms), C.byref(cnt)))
        return ms.value, cnt.value

    fwd_b, bwd_b = algorithmic_bytes(I, O, F)
    # algorithmic bytes of each kernel launch: the tensors that launch has to touch once, tables included
    kernel_bytes = {
        "lut_forward_kernel<6>":  fwd_b,                                         # x, y, W, index table
        "lut_backward_kernel<6>": (4 * F * (I + O) + 3 * 256 * O + 24 * O) if args.dx_mode == 0 else bwd_b,   # x, dy, W, dW (+ dx when fused)
        "lut_dx_kernel<6>":       4 * F * (2 * I + O) + 256 * O + 24 * O,        # x, dy, dx, coefficient and index tables
    }
    kernels = {}
    for which, name in ((0, "lut_forward_kernel<6>"), (1, "lut_backward_kernel<6>"), (3, "lut_dx_kernel<6>")):
        total_ms, launches = read_timer(which)
        if launches == 0:
            continue
        per_step = launches / args.steps
        avg_ms = total_ms / launches
        gbs = kernel_bytes[name] / per_step / (avg_ms * 1e-3) / 1e9
        kernels[name] = {"avg_launch_ms": avg_ms, "launches_per_step": per_step, "algorithmic_bytes_per_launch": kernel_bytes[name] / per_step,
                         "achieved_GBps": gbs, "frac": gbs / HBM_PEAK_GBS}
    dominant = max(kernels, key=lambda k: kernels[k]["avg_launch_ms"] * kernels[k]["launches_per_step"])
    dk = kernels[dominant]
    node_evals = O * F
    ms_per_step = dt / args.steps * 1e3
    out = {
        "metric": "G node-evals/s StochasticLut6 fp32 fwd+bwd (8192 frames x 4096 nodes)",
        "value": node_evals / (dt / args.steps) / 1e9,
        "unit": "G node-evals/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "ms_per_step_with_kernel_events": dt_events / args.steps * 1e3,
        # the per-kernel times below come from the second pass, whose event records (about 3 us each on the device) make it
        # this much slower than the timed region: kernel times sum to slightly more than ms_per_step
        "event_pass_inflation": dt_events / dt,
        "ramp_seconds": ramp_done, "ramp_steps": ramp_steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "StochasticLut6 fwd+bwd fp32, 4096 in x 4096 out x 8192 frames, uniform random 6-of-4096 wiring",
                   "dx_mode": ["deterministic (input-centric, reverse table)", "atomic", "dx_tmp + reverse table"][args.dx_mode],
                   "lut_binarize": False, "binary": False, "frame_stride_floats": S},
        "hbm_frac_step": (fwd_b + bwd_b) / (dt / args.steps) / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": dk["achieved_GBps"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": dk["frac"],
                     "traffic": measured_traffic("kernels", "stochasticlut6/" + dominant.split("<")[0]) if args.dx_mode == 0 else None,
                     "traffic_source": traffic_source()},
        "kernels": kernels,
    }
    if args.profile_copy:
        for _ in range(3):
            y.copy_(x)
        torch.cuda.synchronize()
        out["profile_copy_bytes"] = int(x.numel() * 4)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(I, O, args.cpu_frames, os.cpu_count() if (os.cpu_count() or 1) <= 16 else 16)
    return out


def bench_forward_small(args, lib):
    """BASELINE configuration 1: StochasticLut6 forward only, 784 -> 1024 nodes, 64 frames (the case the reference's CPU path
    runs as is).  Two launches (table preparation, forward) of a few microseconds: the figure is launch latency."""
    import numpy as np
    import torch
    from binarybrain_amd import ops, synth
    I, O, F = 784, 1024, 64
    rng = np.random.default_rng(0)
    S = synth.frame_stride_fp32(F)
    idx_h = synth.wiring(rng, I, O); W_h = synth.lut_tables(rng, O); x_h = synth.uniform_frames(rng, I, F, S)
    idx = torch.from_numpy(idx_h).cuda(); W = torch.from_numpy(W_h).cuda(); x = torch.from_numpy(x_h).cuda()
    y = torch.empty((O, S), device="cuda")

    def step():
        ops.stochastic_lut_forward(6, x, idx, W, F, out=y)

    for _ in range(max(args.warmup, 20)):
        step()
    torch.cuda.synchronize()
    steps = max(args.steps, 200)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    kernel_ms = library_timed_ms(lib, step, steps, 5, which=0)
    nbytes = 4 * F * (I + O) + 280 * O
    out = {"metric": "G node-evals/s StochasticLut6 fp32 forward (784 -> 1024 nodes, 64 frames)", "value": O * F / dt / 1e9,
           "unit": "G node-evals/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 20), "ms_per_step": dt * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "StochasticLut6 forward fp32, 784 in x 1024 out x 64 frames (launch-bound: two launches per call)"},
           "roofline": {"bound": "hbm", "kernel": "lut_forward_kernel<6>", "achieved": nbytes / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                        "unit": "GB/s", "frac": nbytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                        "kernel_ms": kernel_ms}}
    if not args.no_cpu:
        import oracle
        best = None
        for _ in range(20):
            t1 = time.perf_counter()
            if oracle.have_ref():
                oracle.ref_stochastic_lut(6, x_h, idx_h, W_h)
            else:
                oracle.stochastic_lut_forward(6, x_h, idx_h, W_h, F)
            d = time.perf_counter() - t1
            best = d if best is None else min(best, d)
        out["cpu_baseline"] = {"value": O * F / best / 1e9, "unit": "G node-evals/s", "cores": min(os.cpu_count() or 1, 16),
                               "kind": "reference" if oracle.have_ref() else "port",
                               "sample": "the whole configuration (AVX2+OpenMP host Forward incl. the harness's buffer copies), best of 20"}
    return out


def gather_probe_library():
    """bench_gather_probe.so: the bench's own instrumentation kernel, built from bench_gather_probe.hip beside this file
    (by __graft_entry__.build(); here only when it is missing)."""
    import ctypes as C
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    so, src = os.path.join(here, "bench_gather_probe.so"), os.path.join(here, "bench_gather_probe.hip")
    if not os.path.exists(so):
        subprocess.check_call([os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
                               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", src, "-o", so], cwd=here)
    probe = C.CDLL(so)
    probe.bench_row_gather_probe.restype = C.c_int
    probe.bench_row_gather_probe.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 7 + [C.POINTER(C.c_float), C.c_void_p]
    return probe


def bench_gather_ceiling(args, lib):
    """What the GPU sustains on the dx kernel's access pattern alone (instrumentation, a kernel of the bench's own): per (input row,
    128-frame window) 36 pseudo-randomly chosen rows' 512-byte segments are read and discarded — 6 consumers x (5 rows + dy) as in the
    headline shape.  Reported as a rate through L1; the dx kernel moves the same bytes and does its arithmetic on top."""
    import ctypes as C
    import torch
    from binarybrain_amd import synth
    from binarybrain_amd.capi import ptr, stream_ptr
    probe = gather_probe_library()
    I, F = 4096, 8192
    S = synth.frame_stride_fp32(F)
    x = torch.rand((I, S), device="cuda")
    sink = torch.zeros(1, device="cuda")
    loads = 36
    steps, warmup = max(args.steps, 20), max(args.warmup, 20)

    def mean_ms(seg):
        ms = C.c_float(0)
        rc = probe.bench_row_gather_probe(ptr(x), ptr(sink), I, F, S, loads, seg, warmup, steps, C.byref(ms), stream_ptr())
        if rc != 0:
            raise RuntimeError("bench_row_gather_probe failed: %d" % rc)
        return ms.value

    kernel_ms = mean_ms(128)
    nbytes = I * (F // 128) * loads * 512
    # the same bytes as longer or shorter row segments: the rate grows with the bytes per visited row until the window of all rows
    # (4096 rows x segment) no longer fits the 4 MiB L2 of an XCD
    by_segment = {}
    for seg in (64, 128, 256, 512):
        by_segment["%d B" % (seg * 4)] = round(I * (F // seg) * loads * seg * 4 / (mean_ms(seg) * 1e-3) / 1e12, 2)
    return {"metric": "TB/s of gathered 512-byte row segments through L1 (access pattern of the dx kernel, no arithmetic)",
            "value": nbytes / (kernel_ms * 1e-3) / 1e12, "unit": "TB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": kernel_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "row gather probe, 4096 rows x 8192 frames, 36 row segments per (row, 128 frames)", "bytes_per_launch": nbytes,
                       "TBps_by_segment_length": by_segment}}


def other_configs(args, lib):
    """The other BASELINE configurations, measured after the headline workload in the same process: configuration 1 (forward
    784 -> 1024 x 64), 3 (classifier training step), 4 (BinaryLut6 inference), 5 (convolutional block), and the gather
    ceiling that the dx kernel is judged against.  Each entry keeps its own roofline and CPU baseline."""
    import copy
    sub = copy.copy(args)
    sub.ramp_seconds = min(args.ramp_seconds, 0.15)
    sub.profile_copy = False
    keep = ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "config", "roofline", "cpu_baseline")
    out = {}
    for name, fn, workload in (("cfg1_forward_784x1024x64", bench_forward_small, "forward_784x1024x64"),
                               ("cfg3_mnist_step", bench_mnist_step, "mnist_step"),
                               ("cfg4_binarylut6", bench_binarylut6, "binarylut6"),
                               ("cfg5_conv_block", bench_conv_block, "conv_block"),
                               ("dx_gather_ceiling", bench_gather_ceiling, "gather_ceiling")):
        sub.workload = workload
        sub.plain_signatures = False
        r = fn(sub, lib)
        out[name] = {k: r[k] for k in keep if k in r}
        if name in ("cfg3_mnist_step", "cfg5_conv_block"):
            out[name]["ms_per_step_without_hints"] = without_hints(fn, sub, lib)
    sub.workload = "differentiablelut6"
    sub.plain_signatures = False
    r = bench_differentiablelut6(sub, lib)
    out["differentiablelut6_4096x4096x8192"] = {k: r[k] for k in keep if k in r}
    out["differentiablelut6_4096x4096x8192"]["ms_per_step_without_hints"] = without_hints(bench_differentiablelut6, sub, lib)
    return out


def without_hints(fn, args, lib):
    """ms per step of the same workload called as the reference's own classes would call it through include/bbcu_hip_binding.h: the
    reference's signatures only (no bbhip_Hint* call, no entry that folds the table clamp or the gradient clear into another launch)"""
    import copy
    sub = copy.copy(args)
    sub.plain_signatures = True
    sub.no_cpu = True
    return fn(sub, lib)["ms_per_step"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed steps first; the device needs a few dozen steps of load to reach its sustained clock")
    ap.add_argument("--dx-mode", type=int, default=int(os.environ.get("BBHIP_BENCH_DX_MODE", "0")),
                    help="0: deterministic input-centric dx; 1: fp32 atomics; 2: dx_tmp + reverse table")
    ap.add_argument("--separate-clamp", action="store_true",
                    help="headline step: clamp W with a launch of its own (bbhip_fp32_Vector_clamp, then the forward entry) instead of inside the forward entry's table preparation")
    ap.add_argument("--tmp-mb", type=int, default=256,
                    help="dx mode 2: size of the dx_tmp scratch in MiB (the reference caps it at 256; a smaller one takes more passes over shorter frame ranges)")
    ap.add_argument("--ramp-seconds", type=float, default=0.3,
                    help="before the warm-up steps, keep the device under the same load for this long (untimed): from idle it "
                         "takes a few dozen steps to reach its sustained clock, whatever --warmup says")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="headline workload only: skip the other BASELINE configurations that the default run reports under `configs`")
    ap.add_argument("--profile-copy", action="store_true",
                    help="after the timed region, copy x to y three times: a plain copy of known size for calibrating rocprofv3 byte counters")
    ap.add_argument("--workload", default="stochasticlut6", choices=["stochasticlut6", "binarylut6", "differentiablelut6", "differentiablelut6_bit", "mnist_step", "conv_block", "adam", "conv", "tail", "stochastic_bn", "modulation",
                             "forward_784x1024x64", "gather_ceiling"],
                    help="stochasticlut6 (default, the headline metric) or binarylut6 (packed inference, 8192 -> 16384 nodes, 262144 frames)")
    ap.add_argument("--cpu-frames", type=int, default=8192)
    ap.add_argument("--plain-signatures", action="store_true",
                    help="workloads differentiablelut6, mnist_step, conv_block: call the library as the reference's own classes would through "
                         "include/bbcu_hip_binding.h — no bbhip_Hint* call, table clamp and gradient clear as launches of their own")
    ap.add_argument("--write-traffic", metavar="DIR", default=None,
                    help="no benchmark: read the rocprofv3 counter runs under DIR (made by the commands in TRAFFIC_COMMANDS) and write profiles/traffic.json")
    args = ap.parse_args()
    if args.write_traffic:
        write_traffic(args.write_traffic)
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (the path would shard over the "
              "frame axis; no multi-GPU code is built)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from binarybrain_amd import capi, ops, synth

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = capi.lib()
    secondary = {"binarylut6": bench_binarylut6, "adam": bench_adam, "conv": bench_conv, "tail": bench_tail, "stochastic_bn": bench_stochastic_bn, "modulation": bench_modulation,
                 "differentiablelut6": bench_differentiablelut6, "differentiablelut6_bit": bench_differentiablelut6,
                 "mnist_step": bench_mnist_step, "conv_block": bench_conv_block, "forward_784x1024x64": bench_forward_small,
                 "gather_ceiling": bench_gather_ceiling}
    if args.workload in secondary:
        print(json.dumps(secondary[args.workload](args, lib)))
        return
    res = bench_stochasticlut6(args, lib)
    if not args.no_configs:
        res["configs"] = other_configs(args, lib)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
