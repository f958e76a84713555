#!/usr/bin/env python3
"""Benchmark of the convolution hot path on one MI355X.

One "step" is one full DCGAN training iteration at batch 64 in fp32 (BASELINE.json config 3): a
discriminator Adam step on a batch of real and a batch of generated images, then one generator
Adam step, through the operator graph and the HIP backend.  Inputs (z, images, labels) and all
parameters are resident in HBM before the timed region starts; synthetic data, random-init weights.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline      the dominant convolution kernel: algorithmic FLOP/s (HIP events around every launch
                of that kernel inside the timed region, on the stream it is launched on) against the
                fp32 MFMA peak; `kernels` lists every convolution kernel the same way and
                `hbm_kernels` the memory-bound kernels as algorithmic GB/s against the HBM peak
  cpu_baseline  the reference's own CPU operators (oracle/_ref, RT_MODE=CPU arithmetic) timed on this
                host on a bounded sample and extrapolated to one iteration by FLOPs per operator class

`--workload layers` instead sweeps the four DCGAN layer shapes (forward, input gradient, filter
gradient separately; BASELINE.json config 1) at `--batch`, each timed over a sustained run, and
prints one JSON line with a row per (layer, operator).  `--workload generator --batch 4096` times
the generator's forward pass alone (BASELINE.json config 4's inference half; config 0 at batch 64).
`--workload discriminator` times the discriminator's forward and backward pass on labelled images
(BASELINE.json config 2: all dW / db and the gradient of the images, no optimiser).
`cpu_baseline.mcpu` is the reference's RT_MODE=MCPU runtime (4 workers) on the same sample.
`--workload streaming` times the memory-bound operators (bias, activations, their gradients, Adam)
on 128 MiB tensors, as algorithmic GB/s against the HBM peak, with a plain copy beside them.

After the timed region a plain device-to-device copy of 256 MiB runs four times: under
`rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its known size calibrates the counters.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as ge  # noqa: E402

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0
CALIBRATION_COPY_BYTES = 256 << 20

# HBM bytes per launch of the convolution kernels in the batch-64 iteration come from two
# `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE), each scaled by the same counter's
# reading for the calibration copy.  The summary of those runs is kept under profiles/ and is READ here
# (not pasted): regenerating the profile updates the figure, a missing file gives `traffic: null`.
TRAFFIC_SOURCE = "profiles/bench_iteration_bs64_hbm_traffic.md"


def measured_traffic_bytes():
    """{kernel tag: HBM bytes per launch}, launch-weighted over the layer shapes and the single / paired
    instantiations that share a tag, from the table of TRAFFIC_SOURCE (columns: kernel, workgroups,
    launches, FETCH_SIZE KiB, WRITE_SIZE KiB, scaled read MB, scaled write MB, total MB, GB/s)."""
    import re
    path = os.path.join(ROOT, TRAFFIC_SOURCE)
    if not os.path.exists(path):
        return {}
    total, launches = {}, {}
    for line in open(path):
        if not line.startswith("| `"):
            continue
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        name, n, mb = cells[0].strip("`"), int(cells[2]), float(cells[7])
        m = re.match(r"conv_igemm_fast<(\d), (\d+), (\d+), \d, \d(?:, \w+)+>", name)
        tag = ("conv_igemm_fast<%s,%sx%s>" % (("fwd", "dx", "dk")[int(m.group(1))], m.group(2), m.group(3))) if m \
            else name.split("<")[0]
        total[tag] = total.get(tag, 0.0) + n * mb * 1e6
        launches[tag] = launches.get(tag, 0) + n
    return {tag: total[tag] / launches[tag] for tag in total}


# DCGAN layers: (H, W, C, O) of the equivalent forward convolution, 5x5, stride 2, SAME
LAYERS = [(64, 64, 3, 64), (32, 32, 64, 128), (16, 16, 128, 256), (8, 8, 256, 512)]


def hbm_row(r, steps):
    """One memory-bound kernel class of the second pass.  A class whose launches move under 1 MiB (the
    64-element bias gradient of the dense head: 256 bytes) is launch latency and nothing else: it is
    listed with its time and without a bandwidth figure."""
    per_launch = r["flops"] / r["launches"]
    row = {"name": r["name"][4:], "launches": r["launches"], "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
           "bytes_per_launch": round(per_launch), "ms_per_step": round(r["ms"] / steps, 4)}
    if per_launch >= (1 << 20):
        row["gbs"] = round(r["flops"] / (r["ms"] * 1e-3) / 1e9, 3)
        row["frac"] = round(r["flops"] / (r["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
    else:
        row["gbs"] = row["frac"] = None
        row["note"] = "launch-latency bound: %d bytes per launch" % round(per_launch)
    return row


def conv_flops(batch, layer):
    H, W, C, O = layer
    return 2.0 * batch * (H // 2) * (W // 2) * O * 25 * C


def iteration_flops(batch):
    """Algorithmic FLOPs of one iteration by operator class (fwd-type, dx-type, dk-type convs and
    the dense layers).  D step: G fwd, D fwd x2, dk x2, dx (layers 1-3) x2.  G step: G fwd, D fwd,
    D dx (all layers), G dk, G dx (= fwd-type convs of layers 1-3)."""
    f = [conv_flops(batch, l) for l in LAYERS]
    all4, top3 = sum(f), sum(f[1:])
    fwd = 2 * all4 + all4 + top3            # D fwd (2 + 1 times) + G input gradients
    dx = all4 + 2 * top3 + all4 + all4      # G fwd (D step), D dx x2, G fwd (G step), D dx
    dk = 2 * all4 + all4                    # D dk x2, G dk
    dense = 2.0 * batch * (100 * 8192 + 8192) * 3 * 2
    return {"fwd": fwd, "dx": dx, "dk": dk, "dense": dense, "total": fwd + dx + dk + dense}


def synthetic(batch, seed=1234):
    rng = np.random.default_rng(seed)
    pkg = ge.load_package()
    weights = {}
    for name, shape in pkg.hostabi.var_shapes().items():
        if name.endswith("_w"):
            weights[name] = (rng.standard_normal(shape) * 0.02).astype(np.float32)
        else:
            weights[name] = np.zeros(shape, np.float32)
    z = rng.uniform(-1, 1, (batch, 100)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, 64, 64, 3)).astype(np.float32)
    return weights, z, x


def host_cpu():
    """(model name, logical CPUs this process may run on) of the host."""
    name = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                name = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return name, usable


def cpu_baseline(batch):
    """Times the reference's CPU operators (compiled from its own sources into oracle/_ref) on this host:
    conv2d, conv2d_input_grad, conv2d_kernel_grad on layer D1 at batch 4, one thread (RT_MODE=CPU
    arithmetic; about 6 s), and extrapolates one iteration from the measured FLOP/s of each class.
    RT_MODE=MCPU: the reference's rt::optimize + cpu::ThreadPoolRunner on 18 independent nodes of the
    same operators at batch 2, with its own 4 workers (src/ops/graph.cu:32) and with one worker per
    host core this process may use (at most 16, the share of a one-GPU box)."""
    oracle = ge.load_oracle()
    kind = "reference" if oracle.have_ref() else "port"
    orc = oracle.Oracle("ref" if kind == "reference" else "orc")
    orc.set_threads(1)
    cpu_name, usable = host_cpu()
    rng = np.random.default_rng(0)
    H, W, C, O = LAYERS[1]

    def operands(n):
        return (rng.uniform(-1, 1, (n, H, W, C)).astype(np.float32), (rng.standard_normal((5, 5, C, O)) * 0.02).astype(np.float32),
                rng.uniform(-1, 1, (n, H // 2, W // 2, O)).astype(np.float32))

    n = 4
    x, k, dy = operands(n)
    fl = conv_flops(n, LAYERS[1])
    rates = {}
    t0 = time.perf_counter()
    orc.conv2d(x, k, (2, 2))
    rates["fwd"] = fl / (time.perf_counter() - t0)
    t0 = time.perf_counter()
    orc.conv2d_input_grad(dy, k, 2, (H, W))
    rates["dx"] = fl / (time.perf_counter() - t0)
    t0 = time.perf_counter()
    orc.conv2d_kernel_grad(dy, x, 2, (3, 3))
    rates["dk"] = fl / (time.perf_counter() - t0)
    work = iteration_flops(batch)
    seconds = sum(work[c] / rates[c] for c in ("fwd", "dx", "dk")) + work["dense"] / rates["fwd"]
    out = {"value": 1.0 / seconds, "unit": "iterations/s", "cores": 1, "kind": kind, "host_cpu": cpu_name,
           "host_cores_usable": usable,
           "sample": "reference cpu::conv2d / conv2d_input_grad / conv2d_kernel_grad on layer D1 "
                     "([%d,32,32,64] -> 128, 5x5, s2) once each, one thread; iteration time extrapolated "
                     "from the per-class GFLOP/s (%.3f / %.3f / %.3f) over %.0f GFLOP"
                     % (n, rates["fwd"] / 1e9, rates["dx"] / 1e9, rates["dk"] / 1e9, work["total"] / 1e9),
           "gflops": {c: rates[c] / 1e9 for c in rates}}
    if kind != "reference":
        return out
    # RT_MODE=MCPU.  The reference's optimiser leaves convolution nodes whole (src/runtime/optimizer.cu:
    # 239-247, 561-583): what its thread pool gains is the overlap of independent nodes, so the sample is
    # a list of independent nodes -- 6 x (conv2d, input gradient, filter gradient) at batch 2 -- and the
    # speedup over running that list on one thread is an upper bound for a training iteration, whose
    # backward pass offers two to four independent nodes per layer.
    n2, copies = 2, 6
    fl2 = conv_flops(n2, LAYERS[1])
    sequential = copies * sum(fl2 / rates[c] for c in ("fwd", "dx", "dk"))

    def mcpu(workers):
        prog = oracle.RefProgram()
        nodes = []
        for _ in range(copies):
            x2, k2, dy2 = operands(n2)
            nodes += [prog.conv2d(x2, k2, (2, 2), (3, 3))[0], prog.conv2d_input_grad(dy2, k2, 2, (H, W))[0],
                      prog.conv2d_kernel_grad(dy2, x2, 2, (3, 3))[0]]
        t0 = time.perf_counter()
        prog.run(nodes, mcpu=True, workers=workers)
        t = time.perf_counter() - t0
        return {"workers": workers, "sample_seconds": t, "speedup": sequential / t, "value": sequential / t / seconds,
                "unit": "iterations/s"}

    out["mcpu"] = mcpu(4)
    out["mcpu_all_cores"] = mcpu(max(1, min(usable, 16)))
    out["mcpu_value"] = out["mcpu"]["value"]
    out["mcpu_all_cores_value"] = out["mcpu_all_cores"]["value"]
    out["mcpu_all_cores_workers"] = out["mcpu_all_cores"]["workers"]
    out["mcpu_sample"] = ("18 independent nodes (6 x conv2d / input gradient / filter gradient of D1 at batch 2) through the "
                          "reference's rt::optimize + cpu::ThreadPoolRunner; %.1f s on one thread (from the per-class rates); "
                          "iteration rate = one-thread rate x measured speedup, an upper bound" % sequential)
    return out


def calibration_copy(A):
    """A plain copy of known size, for scaling the profiler's memory counters."""
    n = CALIBRATION_COPY_BYTES // 4
    src, dst = A.Buf((n,)), A.Buf((n,))
    lib = A.load()
    A.check(lib.dh_memset0(src.ptr, CALIBRATION_COPY_BYTES, None))
    for _ in range(4):
        A.check(lib.dh_memcpy_d2d(dst.ptr, src.ptr, CALIBRATION_COPY_BYTES, None))
    A.check(lib.dh_sync())


def layer_sweep(args, A):
    """BASELINE.json config 1: every layer shape, forward / input gradient / filter gradient timed
    separately.  Each operator first runs for about 60 ms (clocks settle), then is timed for at
    least 100 ms of back-to-back launches with one pair of HIP events on the launch stream."""
    lib = A.load()
    N = args.batch
    rows = []
    t = A.Timer()
    for li, (H, W, C, O) in enumerate(LAYERS):
        Ho, Wo = H // 2, W // 2
        rng = np.random.default_rng(li)
        x = A.Buf.from_numpy(rng.uniform(-1, 1, (N, H, W, C)).astype(np.float32))
        k = A.Buf.from_numpy((rng.standard_normal((5, 5, C, O)) * 0.02).astype(np.float32))
        dy = A.Buf.from_numpy(rng.uniform(-1, 1, (N, Ho, Wo, O)).astype(np.float32))
        y, dx, dk = A.Buf((N, Ho, Wo, O)), A.Buf((N, H, W, C)), A.Buf((5, 5, C, O))
        ops = {
            "fwd": lambda: A.check(lib.dh_conv2d_fwd(x.ptr, k.ptr, y.ptr, N, H, W, C, 5, 5, O, 2, 2, 1, 1, Ho, Wo,
                                                     None, 0, 0.0, None)),
            "dx": lambda: A.check(lib.dh_conv2d_dx(dy.ptr, k.ptr, dx.ptr, N, Ho, Wo, O, 5, 5, C, 2, 2, 1, 1, H, W,
                                                   None, 0, 0.0, None)),
            "dk": lambda: A.check(lib.dh_conv2d_dk(x.ptr, dy.ptr, dk.ptr, N, H, W, C, Ho, Wo, O, 5, 5, 2, 2, 1, 1,
                                                   None)),
        }
        flops = conv_flops(N, (H, W, C, O))
        for name, fn in ops.items():
            # one bracketed launch tells which kernel runs and what the matrix cores are issued for it
            A.profile_reset()
            A.profile_enable(1)
            fn()
            A.profile_enable(0)
            tagged = A.profile_read()
            issued = sum(r["issued"] for r in tagged) if tagged and all(r["issued"] > 0 for r in tagged) else None
            t.start()
            for _ in range(3):
                fn()
            est = max(t.stop_ms() / 3, 1e-3)
            for _ in range(int(60 / est) + 1):
                fn()
            A.check(lib.dh_sync())
            reps = max(args.steps, int(100 / est) + 1)
            t.start()
            for _ in range(reps):
                fn()
            ms = t.stop_ms() / reps
            tf = flops / (ms * 1e-3) / 1e12
            rows.append({"layer": "D%d" % li, "x": [N, H, W, C], "k": [5, 5, C, O], "op": name, "launches": reps,
                         "kernel": "+".join(r["name"] for r in tagged),
                         "us": round(ms * 1e3, 2), "tflops": round(tf, 2), "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4),
                         "issued_frac": round(issued / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4) if issued else None})
    heavy = [r for r in rows if r["layer"] != "D0"]
    total_fl = sum(conv_flops(N, LAYERS[int(r["layer"][1])]) for r in heavy)
    total_s = sum(r["us"] * 1e-6 for r in heavy)
    tf = total_fl / total_s / 1e12
    worst = min(heavy, key=lambda r: r["frac"])
    print(json.dumps({
        "metric": "conv(_transpose) TFLOP/s as % fp32-MFMA peak (layers D1-D3: forward, input gradient, filter gradient)",
        "value": round(tf, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: DCGAN layer sweep, fp32, batch %d, 5x5 stride 2 SAME; one step = the nine "
                               "operators of layers D1-D3 once each (D0 rows listed, not in value)" % N, "batch": N},
        "device": A.device_info(),
        "roofline": {"kernel": "%s %s" % (worst["layer"], worst["op"]), "bound": "mfma", "achieved": worst["tflops"],
                     "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": worst["frac"],
                     "issued_frac": worst["issued_frac"], "traffic": None,
                     "note": "the slowest of the nine operators; every row is in `layers`; `frac` counts skipped "
                             "padding products as work (it can exceed 1), `issued_frac` is what the matrix cores "
                             "are issued per second against the peak (slice reduction inside the time of both)"},
        "layers": rows,
    }))


def streaming_sweep(args, A):
    """The memory-bound operators of the path (bias add, activations and their gradients, bias
    gradient, add, the Adam kernels) on tensors of `--elements` floats each (default 2^25 = 128 MiB:
    the [512,32,32,64] activation of the batch-512 iteration), where the launch itself no longer
    weighs.  Each operator runs back to back for at least `--sustain-ms` (100 ms; a profiler run
    wants fewer launches) and at least `--steps` launches between one pair of HIP events;
    its rate is algorithmic bytes per launch / time per launch against the 8 TB/s HBM peak.  A plain
    device-to-device copy of the same size (8 B/elem) is timed the same way beside them."""
    import ctypes as C
    lib = A.load()
    n = args.elements
    cols = 64
    rows = n // cols
    n = rows * cols
    rng = np.random.default_rng(7)
    host = rng.uniform(-1, 1, n).astype(np.float32)
    a, b = A.Buf.from_numpy(host), A.Buf.from_numpy(host[::-1].copy())
    o = A.Buf((n,))
    m, v = A.Buf.zeros((n,)), A.Buf.zeros((n,))
    bias = A.Buf.from_numpy(rng.uniform(-1, 1, cols).astype(np.float32))
    db = A.Buf((cols,))
    item = A.AdamItem(p=o.ptr, m=m.ptr, v=v.ptr, g1=a.ptr, g2=None, n=n, lrt=1e-4, g1_parts=0, g2_parts=0)
    items = (A.AdamItem * 1)(item)
    # name, bytes per element, launch
    ops = [
        ("copy (hipMemcpyDtoD)", 8, lambda: lib.dh_memcpy_d2d(o.ptr, a.ptr, n * 4, None)),
        ("bias_add", 8, lambda: lib.dh_bias_add(a.ptr, bias.ptr, o.ptr, rows, cols, None)),
        ("relu", 8, lambda: lib.dh_relu(a.ptr, o.ptr, n, None)),
        ("relu_leaky", 8, lambda: lib.dh_relu_leaky(a.ptr, o.ptr, n, 0.2, None)),
        ("tanh", 8, lambda: lib.dh_tanh(a.ptr, o.ptr, n, None)),
        ("sigmoid", 8, lambda: lib.dh_sigmoid(a.ptr, o.ptr, n, None)),
        ("relu_grad", 12, lambda: lib.dh_relu_grad(a.ptr, b.ptr, o.ptr, n, None)),
        ("leaky_relu_grad", 12, lambda: lib.dh_leaky_relu_grad(a.ptr, b.ptr, o.ptr, 0.2, n, None)),
        ("tanh_grad", 12, lambda: lib.dh_tanh_grad(a.ptr, b.ptr, o.ptr, n, None)),
        ("sigmoid_grad", 12, lambda: lib.dh_sigmoid_grad(a.ptr, b.ptr, o.ptr, n, None)),
        ("add", 12, lambda: lib.dh_add(a.ptr, b.ptr, o.ptr, n, None)),
        ("bias_grad", 4, lambda: lib.dh_bias_grad(a.ptr, db.ptr, rows, cols, None)),
        ("act_bias_grad (leaky)", 12, lambda: lib.dh_act_bias_grad(a.ptr, b.ptr, o.ptr, db.ptr, rows, cols, 2, 0.2, None)),
        ("moment_update", 12, lambda: lib.dh_moment_update(m.ptr, a.ptr, 0.5, 0.5, n, None)),
        ("moment_update2", 12, lambda: lib.dh_moment_update2(v.ptr, a.ptr, 0.999, 0.001, n, None)),
        ("adam_update", 16, lambda: lib.dh_adam_update(o.ptr, m.ptr, v.ptr, 1e-4, 1e-8, n, None)),
        ("adam_step", 28, lambda: lib.dh_adam_step(o.ptr, m.ptr, v.ptr, a.ptr, 0.5, 0.5, 0.999, 0.001, 1e-4, 1e-8, n, None)),
        ("adam_step_multi (1 variable)", 28, lambda: lib.dh_adam_step_multi(items, 1, 0.5, 0.5, 0.999, 0.001, 1e-8, None)),
    ]
    t = A.Timer()
    out_rows = []
    for name, bpe, fn in ops:
        t.start()
        for _ in range(3):
            A.check(fn())
        est = max(t.stop_ms() / 3, 1e-3)
        for _ in range(int(0.3 * args.sustain_ms / est) + 1):
            A.check(fn())
        A.check(lib.dh_sync())
        reps = max(args.steps, int(args.sustain_ms / est) + 1)
        t.start()
        for _ in range(reps):
            A.check(fn())
        ms = t.stop_ms() / reps
        gbs = bpe * n / (ms * 1e-3) / 1e9
        out_rows.append({"op": name, "bytes_per_elem": bpe, "launches": reps, "us": round(ms * 1e3, 2),
                         "gbs": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4)})
    kernels = [r for r in out_rows if not r["op"].startswith("copy")]
    total_b = sum(r["bytes_per_elem"] * n for r in kernels)
    total_s = sum(r["us"] * 1e-6 for r in kernels)
    worst = min(kernels, key=lambda r: r["frac"])
    print(json.dumps({
        "metric": "element-wise / bias / Adam kernels: achieved HBM GB/s (algorithmic bytes) against the 8 TB/s peak",
        "value": round(total_b / total_s / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "the memory-bound operators of the path on tensors of %d floats (%d x %d for the "
                               "bias operators); one step = every operator once" % (n, rows, cols), "elements": n},
        "device": A.device_info(),
        "roofline": {"kernel": worst["op"], "bound": "hbm", "achieved": worst["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": worst["frac"], "traffic": None,
                     "note": "the slowest of the operators; every row is in `operators`, the plain copy beside them"},
        "operators": out_rows,
    }))


def generator_only(args, pkg, A):
    """BASELINE.json config 4, second half (config 0 at --batch 64): the generator's forward pass
    alone -- dense 100 -> 4*4*512, four transpose convolutions with bias and relu / tanh in the
    write-out.  z is resident, the images stay on the device; one step = one pass over the batch."""
    weights, z, _ = synthetic(args.batch)
    model = pkg.hostabi.DcganModel(args.batch, seed=1, mode="GPU")
    model.set_fusion(bool(args.fusion))
    for name, w in weights.items():
        model.set_var(name, w)
    model.set_inputs(z=z)
    for _ in range(args.warmup):
        model.generate(to_host=False)
    model.sync()
    A.profile_reset()
    every = max(1, args.profile_every)
    timer = A.Timer()
    t0 = time.perf_counter()
    timer.start()
    profiled = 0
    for i in range(args.steps):
        on = i % every == 0
        if on:
            A.profile_enable(1)
            profiled += 1
        model.generate(to_host=False)
        if on:
            A.profile_enable(0)
    gpu_ms = timer.stop_ms()
    model.sync()
    wall = time.perf_counter() - t0
    rows = A.profile_read()
    flops = sum(conv_flops(args.batch, l) for l in LAYERS) + 2.0 * args.batch * 100 * 8192
    conv_ms = sum(r["ms"] for r in rows)
    conv_fl = sum(r["flops"] for r in rows)
    dom = max(rows, key=lambda r: r["ms"])
    achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
    print(json.dumps({
        "metric": "DCGAN generator forward images/sec, fp32", "value": round(args.batch * args.steps / wall, 1),
        "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[4] (configs[0] at batch 64): DCGAN generator forward only, fp32, batch %d, "
                               "z dim 100 -> [%d,64,64,3]" % (args.batch, args.batch), "batch": args.batch},
        "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
        "step_gflop": round(flops / 1e9, 2), "step_tflops": round(flops / (wall / args.steps) / 1e12, 3),
        "device": A.device_info(),
        "roofline": {"kernel": dom["name"], "bound": "mfma", "achieved": round(achieved, 3),
                     "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": None,
                     "all_conv_kernels": {"tflops": round(conv_fl / (conv_ms * 1e-3) / 1e12, 3),
                                          "frac": round(conv_fl / (conv_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                                          "ms_per_step": round(conv_ms / max(profiled, 1), 4)},
                     "kernels": [{"name": r["name"], "launches": r["launches"],
                                  "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
                                  "tflops": round(r["flops"] / (r["ms"] * 1e-3) / 1e12, 2),
                                  "issued_frac": round(r["issued"] / (r["ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)
                                  if r["issued"] > 0 else None}
                                 for r in sorted(rows, key=lambda r: -r["ms"])]},
    }))
    model.close()


def discriminator_pass(args, pkg, A):
    """BASELINE.json config 2: the discriminator forward and backward on labelled images (random 0/1 labels) --
    four convolutions with bias and leaky relu, the dense head, sigmoid cross-entropy, and the gradients of all
    ten variables and of the input images, no optimiser (tests/test_dcgan_discriminator.cu:49-136 at batch 64).
    Images and labels are resident, nothing is read back; one step = one pass over the batch."""
    weights, _, x = synthetic(args.batch)
    y = (np.random.default_rng(99).random((args.batch, 1)) < 0.5).astype(np.float32)
    model = pkg.hostabi.DcganModel(args.batch, seed=1, mode="GPU")
    model.set_fusion(bool(args.fusion))
    for name, w in weights.items():
        model.set_var(name, w)
    model.set_inputs(x=x)
    model.set_labels(y)
    for _ in range(args.warmup):
        model.disc_pass(want_loss=False)
    model.sync()
    launches = model.last_launch_count()
    A.profile_reset()
    every = max(1, args.profile_every)
    timer = A.Timer()
    t0 = time.perf_counter()
    timer.start()
    profiled = 0
    for i in range(args.steps):
        on = i % every == 0
        if on:
            A.profile_enable(1)
            profiled += 1
        model.disc_pass(want_loss=False)
        if on:
            A.profile_enable(0)
    gpu_ms = timer.stop_ms()
    model.sync()
    wall = time.perf_counter() - t0
    rows = A.profile_read()
    A.profile_reset()
    A.profile_enable(2)
    aux_steps = max(1, min(20, args.steps))
    for _ in range(aux_steps):
        model.disc_pass(want_loss=False)
    model.sync()
    A.profile_enable(False)
    aux_rows = A.profile_read()
    loss = model.disc_pass()
    # forward, filter gradient and input gradient of all four layers (the images' gradient included) + dense head
    flops = 3 * sum(conv_flops(args.batch, l) for l in LAYERS) + 3 * 2.0 * args.batch * 8192
    conv_ms = sum(r["ms"] for r in rows)
    conv_fl = sum(r["flops"] for r in rows)
    dom = max(rows, key=lambda r: r["ms"])
    achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
    hbm_rows = [r for r in aux_rows if r["name"].startswith("hbm:")]
    print(json.dumps({
        "metric": "DCGAN discriminator forward+backward passes/sec, fp32", "value": round(args.steps / wall, 2),
        "unit": "passes/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[2]: DCGAN discriminator forward + backward, fp32, batch %d, images [%d,64,64,3] "
                               "~ U(-1,1), random 0/1 labels, gradients of all weights and of the images"
                               % (args.batch, args.batch), "batch": args.batch, "fusion": bool(args.fusion)},
        "gpu_ms_per_step": round(gpu_ms / args.steps, 4), "launches_per_step": launches, "loss": float(loss),
        "step_gflop": round(flops / 1e9, 2), "step_tflops": round(flops / (wall / args.steps) / 1e12, 3),
        "images_per_s": round(args.batch * args.steps / wall, 1),
        "device": A.device_info(),
        "roofline": {"kernel": dom["name"], "bound": "mfma", "achieved": round(achieved, 3),
                     "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": None,
                     "all_conv_kernels": {"tflops": round(conv_fl / (conv_ms * 1e-3) / 1e12, 3),
                                          "frac": round(conv_fl / (conv_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                                          "ms_per_step": round(conv_ms / max(profiled, 1), 4)},
                     "kernels": [{"name": r["name"], "launches": r["launches"],
                                  "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
                                  "tflops": round(r["flops"] / (r["ms"] * 1e-3) / 1e12, 2),
                                  "frac": round(r["flops"] / (r["ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                                  "issued_frac": round(r["issued"] / (r["ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)
                                  if r["issued"] > 0 else None}
                                 for r in sorted(rows, key=lambda r: -r["ms"])],
                     "hbm_kernels": [hbm_row(r, aux_steps) for r in sorted(hbm_rows, key=lambda r: -r["ms"])]},
    }))
    model.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--fusion", type=int, default=1)
    ap.add_argument("--workload", choices=["iteration", "layers", "generator", "discriminator", "streaming"], default="iteration")
    ap.add_argument("--elements", type=int, default=1 << 25, help="floats per tensor of --workload streaming")
    ap.add_argument("--sustain-ms", type=float, default=100.0,
                    help="--workload streaming: time each operator over at least this long a run of launches")
    ap.add_argument("--profile-every", type=int, default=10,
                    help="bracket the convolution launches with HIP events in every n-th timed iteration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-drop-in", action="store_true",
                    help="skip the two extra passes that time the table runner and the list-only plan (profiling runs)")
    ap.add_argument("--host-inputs", action="store_true",
                    help="copy z and the image batch from host memory in every iteration (the PCIe-inclusive "
                         "rate; the default keeps them resident)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")

    pkg = ge.load_package()
    A = pkg.hipabi
    if args.workload == "layers":
        layer_sweep(args, A)
        return
    if args.workload == "generator":
        generator_only(args, pkg, A)
        return
    if args.workload == "discriminator":
        discriminator_pass(args, pkg, A)
        return
    if args.workload == "streaming":
        streaming_sweep(args, A)
        return
    weights, z, x = synthetic(args.batch)
    model = pkg.hostabi.DcganModel(args.batch, seed=1, mode="GPU")
    model.set_fusion(bool(args.fusion))
    for name, w in weights.items():
        model.set_var(name, w)
    model.set_inputs(z, x)   # resident from here on

    def iteration():
        if args.host_inputs:         # inputs handed to the runs from pageable host memory, as the reference's loop does
            model.d_step(want_loss=False, z=z, x=x)
            model.g_step(want_loss=False, z=z)
            return
        model.d_step(want_loss=False)
        model.g_step(want_loss=False)

    for _ in range(args.warmup):
        iteration()
    model.sync()

    # Per-kernel timing inside the timed region: the convolution launches of every n-th iteration are
    # bracketed by HIP events on their stream.  Bracketing every iteration costs ~8 % of the iteration
    # (two event records per launch stall the queue between dependent kernels), one in five ~1.5 %, one in ten
    # ~0.7 %; the per-kernel rates come out the same from 55, 110 or 220 launches of the dominant kernel.
    A.profile_reset()
    every = max(1, args.profile_every)
    timer = A.Timer()           # events on the stream the kernels run on (the default stream)
    t0 = time.perf_counter()
    timer.start()
    profiled = 0
    for i in range(args.steps):
        on = i % every == 0
        if on:
            A.profile_enable(1)
            profiled += 1
        iteration()
        if on:
            A.profile_enable(0)
    gpu_ms = timer.stop_ms()    # waits for the stop event
    model.sync()
    wall = time.perf_counter() - t0
    A.profile_enable(False)
    rows = A.profile_read()

    # second, untimed pass: every kernel bracketed (the events of ~150 small launches per iteration
    # would slow the timed region itself, so the memory-bound kernels are measured here)
    A.profile_reset()
    A.profile_enable(2)
    aux_steps = max(1, min(20, args.steps))
    for _ in range(aux_steps):
        iteration()
    model.sync()
    A.profile_enable(False)
    aux_rows = A.profile_read()
    d_loss = model.eval("d_loss")[0]
    g_loss = model.eval("g_loss")[0]

    # the reference's own loop (dcgan/main.cu:378-397): z and the image batch fed from host memory and
    # both losses read back in every iteration -- reported beside the resident rate, never as `value`
    ref_steps = max(1, min(args.steps, 50))
    for _ in range(3):
        model.d_step(z=z, x=x), model.g_step(z=z)
    t1 = time.perf_counter()
    for _ in range(ref_steps):
        model.d_step(z=z, x=x)     # graph.run({d_opti, d_loss}, {z, x}) and the loss read back
        model.g_step(z=z)          # graph.run({g_opti, g_loss}, {z}) and the loss read back
    ref_wall = time.perf_counter() - t1
    # ... and as the reference APPLICATION runs it: the G step twice per iteration (dcgan/main.cu:388-393;
    # BASELINE's configuration, and every other figure of this line, has one)
    t1 = time.perf_counter()
    for _ in range(ref_steps):
        model.d_step(z=z, x=x)
        model.g_step(z=z)
        model.g_step(z=z)
    app_wall = time.perf_counter() - t1

    # What a drop-in behind the reference's seams gets, under the conditions of `value` (inputs resident, no
    # loss read back): node by node through the kernel table (the shim that replaces src/gpu/kernels.cu and
    # runner.cu, nothing else), and the planner when Graph::run hands it the instruction list and nothing
    # else -- gpu::run's own signature -- so that it has to keep every intermediate tensor.  `value` is the
    # planner with the tensors read back named by Graph::run (one added call in src/ops/graph.cu).
    def rate(setup):
        setup()
        for _ in range(3):
            iteration()
        model.sync()
        t = time.perf_counter()
        for _ in range(ref_steps):
            iteration()
        model.sync()
        return ref_steps / (time.perf_counter() - t)

    table_rate = list_only_rate = table_launches = list_only_launches = None
    if not args.no_drop_in:
        table_rate = rate(lambda: model.set_fusion(False))
        table_launches = model.last_launch_count()
        list_only_rate = rate(lambda: (model.set_fusion(True), model.set_name_results(False)))
        list_only_launches = model.last_launch_count()
        model.set_name_results(True)
        model.set_fusion(bool(args.fusion))

    calibration_copy(A)

    ms_per_step = wall * 1e3 / args.steps
    work = iteration_flops(args.batch)
    hbm_rows = [r for r in aux_rows if r["name"].startswith("hbm:")]
    dense_rows = [r for r in aux_rows if r["name"] == "dense gemm"]
    conv_ms = sum(r["ms"] for r in rows)
    conv_fl = sum(r["flops"] for r in rows)
    dom = max(rows, key=lambda r: r["ms"])
    achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
    traffic = measured_traffic_bytes().get(dom["name"]) if args.batch == 64 else None
    if args.batch == 64 and traffic is None:
        print("bench.py: %s has no row for %s; roofline.traffic is null" % (TRAFFIC_SOURCE, dom["name"]), file=sys.stderr)
    traffic = round(traffic) if traffic else None

    def issued_frac(r):
        """Matrix-core utilisation proper: the FLOPs the kernel issues (live k-slabs as full tiles --
        skipped padding taps are not in it) per second against the peak.  The algorithmic `frac` counts
        the skipped products as work done and may exceed it."""
        return round(r["issued"] / (r["ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4) if r["issued"] > 0 else None

    roofline = {
        "kernel": dom["name"], "bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS,
        "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "issued_frac": issued_frac(dom),
        "traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic else None,
        "launches": dom["launches"], "avg_launch_us": round(dom["ms"] * 1e3 / dom["launches"], 2),
        "flops_per_launch": dom["flops"] / dom["launches"],
        "issued_flops_per_launch": dom["issued"] / dom["launches"] if dom["issued"] > 0 else None,
        "all_conv_kernels": {"tflops": round(conv_fl / (conv_ms * 1e-3) / 1e12, 3),
                             "frac": round(conv_fl / (conv_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                             "ms_per_step": round(conv_ms / max(profiled, 1), 4)},
        "profiled_iterations": profiled,
        "kernels": [{"name": r["name"], "launches": r["launches"], "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
                     "tflops": round(r["flops"] / (r["ms"] * 1e-3) / 1e12, 2),
                     "frac": round(r["flops"] / (r["ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                     "issued_frac": issued_frac(r)} for r in sorted(rows, key=lambda r: -r["ms"])],
        "hbm_kernels": [hbm_row(r, aux_steps) for r in sorted(hbm_rows, key=lambda r: -r["ms"])],
        "dense_gemm": [{"launches": r["launches"], "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
                        "ms_per_step": round(r["ms"] / aux_steps, 4)} for r in dense_rows],
        "hbm_kernels_note": "measured in %d extra iterations after the timed region, algorithmic bytes / "
                            "event-bracketed launch time (includes the launch gap)" % aux_steps,
    }
    out = {
        "metric": "DCGAN train iters/sec @bs64 fp32; conv(_transpose) TFLOP/s as % fp32-MFMA peak",
        "value": round(args.steps / wall, 3), "unit": "iterations/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[3]: full DCGAN training iteration (D step on real+fake, one G step, Adam), "
                               "fp32, batch %d, 64x64x3 images, z dim 100" % args.batch,
                   "batch": args.batch, "fusion": bool(args.fusion),
                   "inputs": "copied from host memory every iteration" if args.host_inputs else "resident in HBM"},
        "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
        "iteration_gflop": round(work["total"] / 1e9, 2),
        "iteration_tflops": round(work["total"] / (wall / args.steps) / 1e12, 3),
        "losses_after": {"d_loss": float(d_loss), "g_loss": float(g_loss)},
        "reference_loop_value": round(ref_steps / ref_wall, 3),
        "reference_loop": {"value": round(ref_steps / ref_wall, 3), "unit": "iterations/s", "steps": ref_steps,
                           "ms_per_step": round(ref_wall * 1e3 / ref_steps, 4),
                           "what": "the reference's own training loop (dcgan/main.cu:378-397): z and the image batch fed "
                                   "from pageable host memory and both losses read back in every iteration; one G step "
                                   "per iteration as in BASELINE's configuration",
                           "two_g_steps_value": round(ref_steps / app_wall, 3),
                           "two_g_steps_what": "the same loop with the G step run twice per iteration, as the reference "
                                               "application does (dcgan/main.cu:388-393)"},
        "table_runner_value": round(table_rate, 3) if table_rate else None,
        "drop_in": None if args.no_drop_in else {
            "unit": "iterations/s", "steps": ref_steps,
            "table_runner": {"value": round(table_rate, 3), "launches_in_g_step": table_launches,
                             "what": "every instruction through hip::kernels_list[node->type], in list order, one "
                                     "wait per run: the shim for src/gpu/kernels.cu + runner.cu and no other change"},
            "planner_list_only": {"value": round(list_only_rate, 3), "launches_in_g_step": list_only_launches,
                                  "what": "hip::run(NodesList&) as src/ops/graph.cu:199 calls gpu::run, nothing said "
                                          "about the tensors read afterwards: only fusions that keep every tensor"},
            "planner_results_named": {"value": round(args.steps / wall, 3),
                                      "what": "`value`: Graph::run names the tensors it reads back "
                                              "(hip::set_protected_tensors) before the run"}},
        "device": A.device_info(),
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.batch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
