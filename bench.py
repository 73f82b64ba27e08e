#!/usr/bin/env python3
"""Benchmark of the edge tensor-product hot path on one MI355X.

Default workload (``edge_fwd_bwd``): the lmax=2, C=64 edge message-passing step of BASELINE.json —
N=4096 nodes, E=65536 uniformly random edges, per-edge weights (E, 11, 64), fp32 — forward
(gather x[src] -> channel-wise CG tensor product -> scatter-sum to dst) plus full backward (gradients
w.r.t. node features, edge harmonics and per-edge weights).  A "step" is one forward + backward through
the public autograd API on synthetic seeded inputs resident in HBM.  Weight tensors rotate over several
buffers so that consecutive steps cannot be served from the 256 MB last-level cache.

Prints ONE JSON line: throughput in Medges/s, the roofline record of the dominant kernel (backward),
measured with events on the launch stream, and the CPU baseline (the oracle's restatement of the
reference's CPU path, timed on a bounded sample of the same workload).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor figure

def profiled_traffic(workload):
    """HBM bytes per launch of the dominant kernel as a separate ``rocprofv3 --pmc FETCH_SIZE`` / ``WRITE_SIZE`` pair
    of runs measured them (this run cannot read hardware counters itself): parsed from the committed summary
    ``profiles/uvu_seg_sh2_edge_fwd_bwd.md`` (table row ``| backward | fetched MB | written MB | total MB | ...``).
    Returns (bytes or None, where the figure comes from)."""
    path = os.path.join(ROOT, "profiles", "uvu_seg_sh2_edge_fwd_bwd.md")
    row = {"edge_fwd_bwd": "backward", "edge_fwd": "forward"}.get(workload)
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 4 and cells[0] == row:
                    return int(float(cells[3]) * 1e6), ("profiles/uvu_seg_sh2_edge_fwd_bwd.md (rocprofv3 --pmc "
                                                        "FETCH_SIZE / WRITE_SIZE, separate runs, scaled by the copy kernel)")
    except (OSError, ValueError):
        pass
    return None, "no counter run on record"


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel, measured now: this script is run four times as a child process
    under ``rocprofv3 --pmc`` (one counter per run: FETCH_SIZE, WRITE_SIZE; the workload with a few steps, and the
    streaming copy of 1 GiB whose true traffic is known and gives the scale of each counter).  The backward's figure
    includes its fix-up kernel.  Returns (bytes or None, description)."""
    import csv, glob, shutil, subprocess, tempfile
    if shutil.which("rocprofv3") is None:
        return None, "rocprofv3 not found"
    me = os.path.abspath(__file__)
    # the interpreter binary itself goes after "--": no launcher, shell or env hop between the profiler and the program
    interpreter = os.path.realpath(sys.executable)
    runs = {"work": ["--workload", workload, "--no-cpu-baseline", "--no-configs", "--no-measure-traffic", "--steps", "5",
                     "--warmup", "2", "--kernel-reps", "5"],
            "copy": ["--workload", "copy", "--steps", "5", "--warmup", "2"]}
    env = dict(os.environ, TMPDIR="/tmp")
    raw = {}
    out_dir = tempfile.mkdtemp(prefix="cgtp_pmc_", dir="/tmp")
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            for tag, extra in runs.items():
                d = os.path.join(out_dir, f"{counter}_{tag}")
                cmd = ["timeout", "-s", "KILL", "90", "rocprofv3", "--pmc", counter, "--output-format", "csv",
                       "-d", d, "-o", "t", "--", interpreter, me, *extra]
                res = subprocess.run(cmd, cwd="/tmp", env=env, capture_output=True, text=True)
                files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
                if res.returncode != 0 or not files:
                    return None, f"counter run failed ({counter}, {tag}, exit {res.returncode})"
                acc = {}
                with open(files[0]) as f:
                    for row in csv.DictReader(f):
                        if row["Counter_Name"] != counter:
                            continue
                        for key in ("uvu_seg_bwd_kernel", "uvu_seg_fwd_kernel", "uvu_fixup_kernel", "copy_kernel"):
                            if key in row["Kernel_Name"]:
                                acc.setdefault(key, []).append(float(row["Counter_Value"]))
                raw[(counter, tag)] = {k: sum(v) / len(v) for k, v in acc.items()}
    finally:
        shutil.rmtree(out_dir, ignore_errors=True)
    try:
        gib_kib = float(1 << 20)                                   # the copy kernel reads and writes 1 GiB
        scale = {c: gib_kib / raw[(c, "copy")]["copy_kernel"] for c in ("FETCH_SIZE", "WRITE_SIZE")}
        names = ["uvu_seg_bwd_kernel", "uvu_fixup_kernel"] if workload == "edge_fwd_bwd" else ["uvu_seg_fwd_kernel"]
        kib = sum(raw[(c, "work")].get(n, 0.0) * scale[c] for c in scale for n in names)
    except (KeyError, ZeroDivisionError):
        return None, "counter run gave no rows for the kernels"
    return int(kib * 1024), ("measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE in child processes, scaled by "
                             f"the copy kernel (x{scale['FETCH_SIZE']:.3f} / x{scale['WRITE_SIZE']:.3f})")


WORKLOADS = {
    # name: (lmax, channels, nodes, edges)
    "edge_fwd_bwd": (2, 64, 4096, 65536),
    "edge_fwd": (2, 64, 4096, 65536),
    # BASELINE configs[4]: high-l channel-wise product, forward + backward, on the large-table kernels
    "edge_l6_fwd_bwd": (6, 32, 20000, 200000),
    # fully connected product on the matrix cores (BASELINE configs[3]): (lmax, C_in = C_out, batch)
    "uvw_fwd": (3, 128, 32768),
    "uvw_fwd_bwd": (3, 128, 32768),
    # the same products in fp32 on the table-driven matrix-core kernels: SO3Linear('uv') at the configs[3] shape, and
    # TensorProduct('uvw') with (lmax, U = V = W, batch)
    "u1v_fp32_fwd_bwd": (3, 128, 32768),
    "uvw_fp32_fwd_bwd": (2, 32, 32768),
    # SO3Linear('uv') with a weight per sample on the streaming kernels: (lmax, C_in = C_out, batch); W is 738 MB
    "u1v_per_sample_fwd_bwd": (2, 16, 65536),
    # the edge step for irreps without a compiled table (0e+1o+2e+3o <- 1o+2e+3o x 0e+1o+2e), fused table-driven kernels
    "edge_table_fwd_bwd": (None, 64, 4096, 65536),
    # the headline edge workload with the per-edge weights formed inside the kernels from 16 features per edge
    "edge_radial_fwd_bwd": (2, 64, 4096, 65536),
    # streaming kernels of known traffic (1 GiB): counter calibration and achievable-bandwidth reference
    "copy": None,
    "read": None,
    # indexed scale-segment reduction alone: the messages of BASELINE configs[1] summed to their destination nodes
    "scatter": None,
    # spherical harmonics of 2^20 vectors up to degree 6 (forward and gradient kernels), normalisation fused
    "sh": None,
    # IrrepsLinear 128 -> 128 channels on 32768 x (0e+1o+2e+3o), bf16, shared weight, forward + backward
    "irreps_linear": None,
    # element-wise and SO(2) modules on 65536 rows of 0e+1o+2e, 64 channels, fp32 (table of timings)
    "modules": None,
    # a whole message-passing layer (harmonics + radial MLP + fused edge product + mixing + gate + layer norm) at the
    # shape of BASELINE configs[2], forward + backward, launched eagerly and replayed as one recorded HIP graph
    "layer": None,
    # plain library GEMM (torch.matmul, bf16, 8192^3): the matrix rate the box reaches, next to the vendor peak
    "gemm": None,
}


def gemm_bench(steps, warmup):
    """bf16 8192 x 8192 x 8192 torch.matmul (hipBLASLt): achievable dense matrix rate on this box."""
    dev = torch.device("cuda:0")
    n = 8192
    a = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    b = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    for _ in range(warmup):
        a @ b
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        a @ b
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    tf = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    print(json.dumps({"metric": "bf16 GEMM TFLOP/s (8192^3, torch.matmul)", "value": round(tf, 1), "unit": "TFLOP/s",
                      "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
                      "data": "synthetic", "config": {"workload": "gemm: library GEMM, calibration of the MFMA peak"},
                      "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                                   "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}}))


def sh_bench(steps, warmup):
    """SphericalHarmonics(l_max=6, normalize_input=True) forward and its gradient on 2^20 vectors: a step is one
    forward and one backward launch through the C ABI.  Per vector the forward reads 12 B and writes 196 B, the
    backward reads 12 + 196 B and writes 12 B."""
    from equitorch_amd import _lib
    dev = torch.device("cuda:0")
    n, lmax = 1 << 20, 6
    d = (lmax + 1) ** 2
    gen = torch.Generator().manual_seed(0)
    v = torch.randn(n, 3, generator=gen).to(dev)
    g = torch.randn(n, d, generator=gen).to(dev)
    y, gv = torch.empty(n, d, device=dev), torch.empty(n, 3, device=dev)
    st = _lib.stream_ptr(dev)
    fwd = lambda: _lib.check(_lib.lib.cgtp_sh_forward(v.data_ptr(), y.data_ptr(), n, lmax, 1, 1.0, _lib.F32, st))
    bwd = lambda: _lib.check(_lib.lib.cgtp_sh_backward(v.data_ptr(), g.data_ptr(), gv.data_ptr(), n, lmax, 1, 1.0,
                                                       _lib.F32, st))

    def timed(fn):
        evs = []
        for _ in range(steps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs) / len(evs)

    for _ in range(warmup):
        fwd(); bwd()
    f_ms, b_ms = timed(fwd), timed(bwd)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fwd(); bwd()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    f_bytes, b_bytes = n * (3 + d) * 4, n * (6 + d) * 4
    gbs = f_bytes / (f_ms * 1e-3) / 1e9
    # CPU baseline: the oracle's restatement of the reference recursion, forward + autograd backward, on a sample
    from oracle import ref_sh
    sample = 1 << 17
    vc = v[:sample].cpu().double().requires_grad_(True)
    gc = g[:sample].cpu().double()
    ref_sh.spherical_harmonics(ref_sh.normalize(vc[:16]), lmax)
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 10.0:
        torch.autograd.grad(ref_sh.spherical_harmonics(ref_sh.normalize(vc), lmax), vc, gc)
        reps += 1
    cpu = {"value": round(sample * reps / (time.perf_counter() - t0) / 1e6, 3), "unit": "Mvectors/s",
           "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"{sample} of the {n} vectors, oracle ref_sh (float64 torch) forward + autograd backward, {cpu_model()}"}
    print(json.dumps({"cpu_baseline": cpu, "metric": "spherical harmonics fwd+bwd Mvectors/s (lmax=6)", "value": round(n / (ms * 1e-3) / 1e6, 1),
                      "unit": "Mvectors/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"sh: {n} vectors, degrees 0..{lmax}, input normalised in the kernel"},
                      "roofline": {"bound": "hbm", "kernel": "cgtp::sh_kernel<float,false,6>", "achieved": round(gbs, 1),
                                   "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                                   "traffic": None, "algorithmic_bytes": f_bytes, "avg_ms": round(f_ms, 5)},
                      "kernels": {"fwd_avg_ms": round(f_ms, 5), "fwd_GBs": round(gbs, 1), "bwd_avg_ms": round(b_ms, 5),
                                  "bwd_GBs": round(b_bytes / (b_ms * 1e-3) / 1e9, 1)}}))


def irreps_linear_bench(steps, warmup):
    """IrrepsLinear(0e+1o+2e+3o -> same, 128 -> 128 channels) on 32768 rows in bf16: a step is the forward and the
    gradients of input and weight.  On the matrix-core kernels of the fully connected product (second operand = 1).
    The forward reads x (134 MB) and the weight, writes out (134 MB): HBM-bound at 64 flops per byte."""
    from equitorch_amd.nn import IrrepsLinear
    dev = torch.device("cuda:0")
    irr, n, c = "0e+1o+2e+3o", 32768, 128
    torch.manual_seed(0)
    mod = IrrepsLinear(irr, irr, c, c).to(dev).to(torch.bfloat16)
    d = mod.irreps_in_dim
    x = torch.randn(n, d, c, device=dev).bfloat16().requires_grad_(True)
    ct = torch.randn(n, d, c, device=dev).bfloat16()

    def step():
        return torch.autograd.grad(mod(x), (x, mod.weight), ct)

    def fwd():
        with torch.no_grad():
            return mod(x)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    evs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fwd()
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    f_ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    nbytes = 2 * n * d * c * 2 + mod.weight.numel() * 2
    gbs = nbytes / (f_ms * 1e-3) / 1e9
    flops = 2 * n * d * c * c
    print(json.dumps({"metric": "IrrepsLinear fwd+bwd Mrows/s (lmax=3, 128->128, bf16)", "value": round(n / (ms * 1e-3) / 1e6, 2),
                      "unit": "Mrows/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": f"irreps_linear: {n} rows of {irr}, {c} -> {c} channels, shared weight (4,{c},{c})"},
                      "roofline": {"bound": "hbm", "kernel": "cgtp::uv_kernel<UV_lin_sh3_d0,128> (forward)",
                                   "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes": nbytes,
                                   "avg_ms": round(f_ms, 5), "fwd_TFLOPs": round(flops / (f_ms * 1e-3) / 1e12, 1)}}))


def modules_bench(steps, warmup):
    """Forward and forward + backward times of the element-wise and SO(2) modules on 65536 rows of 0e+1o+2e with 64
    channels in fp32 (151 MB per feature tensor).  ``value`` is LayerRMSNorm forward + backward; the roofline entry is
    its forward launch (reads and writes the feature tensor once); the other modules are listed under ``modules``."""
    import math

    from equitorch_amd import nn as enn
    from equitorch_amd.nn.functional import sincos
    dev = torch.device("cuda:0")
    irr, n, c, d, k = "0e+1o+2e", 65536, 64, 9, 3
    torch.manual_seed(0)
    x = torch.randn(n, d, c, device=dev)
    gates = torch.randn(n, k, c, device=dev)
    sc = [sincos(torch.rand(n, device=dev) * 2 * math.pi, 2) for _ in range(3)]

    def timed(fn, reps):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    def both(mod, *extra):
        xr = x.clone().requires_grad_(True)

        def fwd():
            with torch.no_grad():
                return mod(x, *extra)

        ct = torch.randn_like(fwd())

        def step():
            return torch.autograd.grad(mod(xr, *extra), xr, ct)
        return round(timed(fwd, steps), 5), round(timed(step, steps), 5)

    norm = enn.LayerRMSNorm(irr, c).to(dev)
    table = {
        "LayerRMSNorm": both(norm),
        "Gate": both(enn.Gate(irr, activation=None).to(dev), gates),
        "SquaredNorm": both(enn.SquaredNorm(irr).to(dev)),
        "TensorDot_uu": both(enn.TensorDot(irr, "uu").to(dev), x),
        "Norm": both(enn.Norm(irr).to(dev)),
        "BatchRMSNorm_train": both(enn.BatchRMSNorm(irr, c).to(dev).train()),
        "BatchRMSNorm_eval": both(enn.BatchRMSNorm(irr, c).to(dev).eval()),
        "IrrepsLinear_fp32": both(enn.IrrepsLinear(irr, irr, c, c).to(dev)),
        "IrrepWiseLinear_fp32": both(enn.IrrepWiseLinear(irr, c, c).to(dev)),
        "SO2Linear_uu": both(enn.SO2Linear(irr, irr, c, c, feature_mode="uu").to(dev)),
        "SO2Linear_uv": both(enn.SO2Linear(irr, irr, c, c, feature_mode="uv").to(dev)),
        "SparseWignerRotation": both(enn.SparseWignerRotation(irr).to(dev), *sc),
        "copy": (round(timed(lambda: x.clone(), steps), 5), None),
    }
    f_ms, step_ms = table["LayerRMSNorm"]
    nbytes = 2 * x.numel() * 4 + norm.weight.numel() * 4
    gbs = nbytes / (f_ms * 1e-3) / 1e9
    print(json.dumps({"metric": "LayerRMSNorm fwd+bwd Mrows/s (0e+1o+2e, C=64, fp32)", "value": round(n / (step_ms * 1e-3) / 1e6, 1),
                      "unit": "Mrows/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": step_ms,
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"modules: {n} rows of {irr}, {c} channels"},
                      "roofline": {"bound": "hbm", "kernel": "cgtp::layer_rms_fwd_kernel<float,4>", "achieved": round(gbs, 1),
                                   "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                                   "traffic": None, "algorithmic_bytes": nbytes, "avg_ms": f_ms},
                      "modules": {name: {"fwd_ms": f, "fwd_bwd_ms": fb} for name, (f, fb) in table.items()}}))


def scatter_bench(steps, warmup):
    """`indexed_scale_segment(msg.view(1, E, 576), None, perm, ptr)` at N = 4096, E = 65536 (lmax = 2, C = 64): reads
    every message once (151 MB) and the sorted tables, writes the node rows (9.4 MB)."""
    from equitorch_amd.ops import indexed_scale_segment
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(0)
    n_nodes, n_edges, feat = 4096, 65536, 576
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    perm = torch.sort(dst, stable=True).indices.to(dev)
    ptr = torch.zeros(n_nodes + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(torch.bincount(dst, minlength=n_nodes), 0)
    ptr = ptr.to(dev)
    msgs = [torch.randn(1, n_edges, feat, generator=gen).to(dev) for _ in range(4)]
    for i in range(warmup):
        indexed_scale_segment(msgs[i % 4], None, perm, ptr, out_size=n_nodes)
    evs = []
    for i in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        indexed_scale_segment(msgs[i % 4], None, perm, ptr, out_size=n_nodes)
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    nbytes = n_edges * feat * 4 + n_nodes * feat * 4 + n_edges * 8 + (n_nodes + 1) * 8
    gbs = nbytes / (ms * 1e-3) / 1e9
    print(json.dumps({"metric": "scatter-sum Medges/s (576 floats per edge)", "value": round(n_edges / (ms * 1e-3) / 1e6, 1),
                      "unit": "Medges/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"scatter: indexed_scale_segment of (1, {n_edges}, {feat}) to {n_nodes} nodes"},
                      "roofline": {"bound": "hbm", "kernel": "cgtp::segment_sum_kernel<float,4>", "achieved": round(gbs, 1),
                                   "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                                   "traffic": None, "algorithmic_bytes": nbytes, "avg_ms": round(ms, 5)}}))


def stream_rate(kind, steps, warmup):
    """(GB/s, ms per launch) of a plain 1 GiB device copy (reads 1 GiB, writes 1 GiB) or read on this box."""
    import ctypes
    from equitorch_amd import _lib
    blib = ctypes.CDLL(os.path.join(ROOT, "equitorch_amd", "lib", "libcgtp_bench.so"))
    for fn in (blib.cgtpbench_copy, blib.cgtpbench_read):
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    dev = torch.device("cuda:0")
    n_bytes = 1 << 30
    src = torch.empty(n_bytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty(n_bytes if kind == "copy" else 16, dtype=torch.uint8, device=dev)
    stream = _lib.stream_ptr(dev)

    def launch():
        if kind == "copy":
            _lib.check(blib.cgtpbench_copy(dst.data_ptr(), src.data_ptr(), n_bytes, stream))
        else:
            _lib.check(blib.cgtpbench_read(src.data_ptr(), dst.data_ptr(), n_bytes, stream))
    for _ in range(warmup):
        launch()
    evs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); launch(); b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ms = sum(a.elapsed_time(b) for a, b in evs) / steps
    moved = n_bytes * (2 if kind == "copy" else 1)
    del src, dst
    return moved / ms / 1e6, ms


def membench(kind, steps, warmup):
    """The streaming kernels as a workload of their own; one JSON line with the achieved GB/s."""
    n_bytes = 1 << 30
    gbs, ms = stream_rate(kind, steps, warmup)
    print(json.dumps({"metric": f"membench_{kind}", "value": round(gbs, 1), "unit": "GB/s",
                      "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
                      "bytes_read": n_bytes, "bytes_written": n_bytes if kind == "copy" else 0,
                      "config": {"workload": f"{kind} of 1 GiB, float4 grid-stride, 4096 workgroups"}}))


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix, vendor figure


def uvw_bench(args):
    """BASELINE configs[3], forward: bf16 x (B,16,128), sh (B,16), shared W (23,128,128), fp32 accumulation;
    algorithmic flops 2*B*99*128*128 (the Clebsch-Gordan stage is not counted)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uvw_mfma
    from equitorch_amd.utils._sh import spherical_harmonics
    lmax, ch, n = WORKLOADS[args.workload]
    backward = args.workload == "uvw_fwd_bwd"
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(dev)
    d = (lmax + 1) ** 2
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, d, ch, generator=gen).bfloat16().to(dev)
    vec = torch.randn(n, 3, generator=gen)
    sh = spherical_harmonics(vec / vec.norm(dim=-1, keepdim=True), lmax).bfloat16().to(dev)
    w = (torch.randn(mod.num_paths, ch, ch, generator=gen) / (ch * mod.num_paths) ** 0.5).bfloat16().to(dev)
    cfg = _uvw_mfma.uv_config_of(mod.tp_info_forward)
    wt = _uvw_mfma.pack_weights(0, w, cfg)
    s1 = int(mod.tp_info_forward.info_Mij_fwd.out_size)
    flops = 2.0 * n * s1 * ch * ch
    if backward:
        return uvw_fwd_bwd_bench(args, mod, x, sh, w, cfg, flops, irreps, gen)

    def step():
        return mod(x, sh, w)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3
    evs = []
    for _ in range(args.kernel_reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); _uvw_mfma._apply(cfg, 0, x, sh, wt, d); b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    k_ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    tf = flops / (k_ms * 1e-3) / 1e12
    return ({
        "metric": "uvw fwd TFLOP/s (lmax=3,C=128,bf16)", "value": round(flops / (ms_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"uvw_fwd: B={n}, irreps {irreps}, C_in=C_out={ch}, shared W ({mod.num_paths},{ch},{ch}), "
                               f"bf16 in / fp32 accumulate / bf16 out, forward through SO3Linear('uv')"},
        "roofline": {"bound": "mfma", "kernel": "cgtp::uv_kernel<UV_sh3_d0,128>", "achieved": round(tf, 2),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": None, "algorithmic_flops": flops, "avg_ms": round(k_ms, 5)}})


def uvw_fwd_bwd_bench(args, mod, x, sh, w, cfg, flops, irreps, gen):
    """BASELINE configs[3], forward and backward (gx, gsh, gW).  Each of the four products contracts the 99
    (path, row) tiles with a 128 x 128 weight once, so the step is priced at 4 x the forward's flops."""
    from equitorch_amd.nn.functional import _uvw_mfma
    n, d, ch = x.shape
    ct = torch.randn(n, d, ch, generator=gen).bfloat16().to(x.device)
    xg, shg, wg = (t.clone().requires_grad_(True) for t in (x, sh, w))

    def step():
        out = mod(xg, shg, wg)
        return torch.autograd.grad(out, (xg, shg, wg), ct)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3

    def timed(fn):
        evs = []
        for _ in range(args.kernel_reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(); b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    w0, w1 = _uvw_mfma.pack_weights(0, w, cfg), _uvw_mfma.pack_weights(1, w, cfg)
    kern = {
        "fwd_ms": timed(lambda: _uvw_mfma._apply(cfg, 0, x, sh, w0, d)),
        "grad_x_ms": timed(lambda: _uvw_mfma._apply(cfg, 1, ct, sh, w1, d)),
        "grad_sh_ms": timed(lambda: _uvw_mfma._grad_y(cfg, x, ct, w0, sh.shape[-1])),
        "grad_w_ms": timed(lambda: _uvw_mfma._grad_w(cfg, x, sh, ct)),
    }
    dom = max(kern, key=kern.get)
    tf = flops / (kern[dom] * 1e-3) / 1e12
    names = {"fwd_ms": "cgtp::uv_kernel<UV_sh3_d0,128>", "grad_x_ms": "cgtp::uv_kernel<UV_sh3_d1,128>",
             "grad_sh_ms": "cgtp::uv_gy_kernel<UV_sh3_gy,128>", "grad_w_ms": "cgtp::uv_gw_kernel<UV_sh3_gw>"}
    return ({
        "metric": "uvw fwd+bwd TFLOP/s (lmax=3,C=128,bf16)", "value": round(4 * flops / (ms_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"uvw_fwd_bwd: B={n}, irreps {irreps}, C_in=C_out={ch}, shared W ({w.shape[0]},{ch},{ch}), "
                               f"bf16 in / fp32 accumulate / bf16 out, SO3Linear('uv') forward + grads of x, sh, W"},
        "roofline": {"bound": "mfma", "kernel": names[dom], "achieved": round(tf, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "algorithmic_flops": flops, "avg_ms": round(kern[dom], 5)},
        "kernels": {k: round(v, 5) for k, v in kern.items()}})


def make_inputs(lmax, ch, n_nodes, n_edges, n_rot, device, graph="uniform"):
    """Seeded CPU generation in the fixed order src, dst, x, vec -> sh, W, ct; then moved to the device.
    ``graph='local'`` (not the BASELINE workload): every edge starts within 64 node ids of where it ends, the
    locality a radius graph over spatially ordered atoms has."""
    from equitorch_amd.utils._sh import spherical_harmonics
    gen = torch.Generator().manual_seed(0)
    d = (lmax + 1) ** 2
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    if graph == "local":
        src = (dst + torch.randint(-64, 65, (n_edges,), generator=gen)) % n_nodes
    x = torch.randn(n_nodes, d, ch, generator=gen)
    vec = torch.randn(n_edges, 3, generator=gen)
    sh = spherical_harmonics(vec / vec.norm(dim=-1, keepdim=True), lmax)
    return dict(src=src, dst=dst, x=x, sh=sh, gen=gen, d=d)


def algorithmic_bytes(n_nodes, n_edges, d, p, ch):
    """Compulsory HBM traffic of one launch: every distinct input byte once, every output byte once, int64
    index tables as in the reference."""
    f = 4
    w = n_edges * p * ch * f
    node = n_nodes * d * ch * f
    edge_sh = n_edges * d * f
    idx = 2 * n_edges * 8 + (n_nodes + 1) * 8
    fwd = w + node + edge_sh + node + idx            # read W, x, sh, tables; write out
    bwd = (w + node + node + edge_sh + idx) + (w + edge_sh + node)  # read W, ct, x, sh, tables; write gW, gsh, gx
    return fwd, bwd


FP32_VECTOR_PEAK_TFLOPS = 157.3  # MI355X fp32, vendor figure (packed instructions: two values per lane and issue)
FP32_UNPACKED_PEAK_TFLOPS = 78.6  # the same with one value per lane: what code built with packed fp32 off can issue at most
# per the data sheet; a register-only loop of independent v_fma_f32 on this chip issues one every 1.15 ns per SIMD from
# two wavefronts per SIMD up (2.07 ns from one): 114 TFLOP/s over 1024 SIMDs
FP32_MEASURED_ISSUE_TFLOPS = 114.0


def edge_rows_bench(args):
    """BASELINE configs[4] (lmax = 6, C = 32, N = 20000, E = 200000, per-edge weights), forward + backward.  The
    table (6460 coefficients) runs on the large-table row kernels: messages and per-edge input gradients go through
    memory and are summed by the segment-sum kernel.  The arithmetic dominates here: about two vector instructions
    per coefficient and channel, priced as 2 * (T + S1) * C flops per edge forward and three times that backward
    (T coefficients, S1 = 826 (path, row) weight products)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    lmax, ch, n_nodes, n_edges = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(dev)
    p = mod.num_paths
    n_rot = min(args.rotate, 2)
    inp = make_inputs(lmax, ch, n_nodes, n_edges, n_rot, dev)
    d = inp["d"]
    plan = EdgePlan(inp["src"].to(dev), inp["dst"].to(dev), n_nodes)
    x = inp["x"].to(dev).requires_grad_(True)
    sh = inp["sh"].to(dev).requires_grad_(True)
    ws = [torch.randn(n_edges, p, ch, generator=inp["gen"]).to(dev).requires_grad_(True) for _ in range(n_rot)]
    ct = torch.randn(n_nodes, d, ch, generator=inp["gen"]).to(dev)

    def step(i):
        w = ws[i % n_rot]
        out = edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward)
        return torch.autograd.grad(out, (x, sh, w), ct)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3

    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    xd, shd = x.detach(), sh.detach()

    def timed(fn):
        evs = []
        for i in range(max(3, args.kernel_reps // 3)):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            w = ws[i % n_rot].detach()
            a.record(); fn(w); b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    # the launches of the step: gather, product and segment sum fused (kernel + fix-up of the cut segments)
    fwd_ms = timed(lambda w: kernels.uvu_forward(cfg, dims, xd, shd, w, seg=plan.fwd_index))
    bwd_ms = timed(lambda w: kernels.uvu_backward(cfg, dims, xd, shd, w, ct, (True, True, True), seg=plan.bwd_index))
    # for comparison: the same products per edge row, without the segment sums that would have to follow
    rows_fwd_ms = timed(lambda w: kernels.uvu_forward(cfg, dims, xd, shd, w, gather=plan.src))
    rows_bwd_ms = timed(lambda w: kernels.uvu_backward(cfg, dims, xd, shd, w, ct, (True, True, True), gather=plan.dst,
                                                       x_gather=plan.src))
    nnz, s1 = dims[4], int(mod.tp_info_forward.info_Mij_fwd.out_size)
    flops_fwd = 2.0 * (nnz + s1) * ch * n_edges
    fwd_bytes, bwd_bytes = algorithmic_bytes(n_nodes, n_edges, d, p, ch)
    msg = 0                     # per-edge rows stay in LDS
    tf = 3 * flops_fwd / (bwd_ms * 1e-3) / 1e12
    gbs = (bwd_bytes + msg) / (bwd_ms * 1e-3) / 1e9
    rec = {
        "metric": "edge-TP fwd+bwd Medges/s (lmax=6,C=32)", "value": round(n_edges / (ms_step * 1e-3) / 1e6, 2),
        "unit": "Medges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: N={n_nodes} nodes, E={n_edges} edges, irreps {irreps}, C={ch}, "
                               f"per-edge weights (E,{p},{ch}), {n_rot} rotating weight buffers"},
        "roofline": {"bound": "hbm", "kernel": "cgtp::uvu_big_seg_bwd_kernel<TPB_sh6,1>", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes": bwd_bytes + msg, "avg_ms": round(bwd_ms, 4),
                     "fp32_vector": {"achieved": round(tf, 2), "peak": FP32_VECTOR_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(tf / FP32_VECTOR_PEAK_TFLOPS, 4),
                                     "unpacked_peak": FP32_UNPACKED_PEAK_TFLOPS,
                                     "frac_of_unpacked": round(tf / FP32_UNPACKED_PEAK_TFLOPS, 4),
                                     "measured_issue_rate": FP32_MEASURED_ISSUE_TFLOPS,
                                     "frac_of_measured_issue_rate": round(tf / FP32_MEASURED_ISSUE_TFLOPS, 4),
                                     "algorithmic_flops": 3 * flops_fwd}},
        "kernels": {"fwd_ms": round(fwd_ms, 4), "bwd_ms": round(bwd_ms, 4),
                    "rows_fwd_ms": round(rows_fwd_ms, 4), "rows_bwd_ms": round(rows_bwd_ms, 4),
                    "fwd_TFLOPs": round(flops_fwd / (fwd_ms * 1e-3) / 1e12, 2),
                    "fwd_fp32_frac_of_unpacked": round(flops_fwd / (fwd_ms * 1e-3) / 1e12 / FP32_UNPACKED_PEAK_TFLOPS, 4),
                    "fwd_GBs": round((fwd_bytes + msg) / (fwd_ms * 1e-3) / 1e9, 1)},
    }
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(inp, lmax, ch, n_nodes, min(args.cpu_sample_edges, 1024))
    return rec


def cpu_baseline(inp, lmax, ch, n_nodes, sample_edges, budget_s=12.0):
    """The oracle's step-for-step restatement of the reference's CPU path (index_select -> product -> scale ->
    CSR segment-sum; forward and backward), timed on the first ``sample_edges`` edges of the same graph."""
    from oracle import ref_ops, ref_tables
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    fwd, b1, b2, n_paths = ref_tables.tp_infos(irreps, irreps, irreps)
    fwd, b1, b2 = (ref_ops.tables_to_torch(t) for t in (fwd, b1, b2))
    e = sample_edges
    src, dst = inp["src"][:e], inp["dst"][:e]
    scale_fwd, _ = ref_tables.sparse_scale_infos(index=list(range(e)), index_out=dst.tolist(),
                                                 out_size=n_nodes, in_size=e)
    perm = torch.tensor(scale_fwd["index"]) if scale_fwd["index"] is not None else None
    ptr = torch.tensor(scale_fwd["seg_out"])
    gen = torch.Generator().manual_seed(1)
    x, sh = inp["x"], inp["sh"][:e]
    w = torch.randn(e, n_paths, ch, generator=gen)
    ct = torch.randn(n_nodes, inp["d"], ch, generator=gen)

    def step():
        out, inter = ref_ops.cpu_edge_forward(x, sh, w, src, perm, ptr, fwd)
        return out, ref_ops.cpu_edge_backward(ct, x, sh, w, inter, src, dst, fwd, b1, b2)

    step()
    t0 = time.perf_counter()
    step()
    one = time.perf_counter() - t0
    iters = max(2, min(20, int(budget_s / max(one, 1e-3))))
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(e / med / 1e6, 4), "unit": "Medges/s", "cores": threads, "kind": "port",
            "sample": f"first {e} of {inp['src'].shape[0]} edges of the same graph, fwd+bwd, median of {iters} "
                      f"runs, {med * 1e3:.1f} ms/run, torch {torch.__version__} CPU ops, {threads} threads on "
                      f"{cpu_model()} ({os.cpu_count()} logical CPUs)"}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def layer_bench(steps, warmup):
    """Forward + backward of a message-passing layer built from the public modules on 4096 nodes / 65536 edges,
    0e+1o+2e, 64 channels, fp32: wall time per step launched eagerly from Python, and the same step recorded once
    with ``torch.cuda.graph`` and replayed (the launches are host-bound when issued one by one)."""
    import time

    from equitorch_amd import nn as enn
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu_radial, edge_tensor_product_uu_vectors
    dev = torch.device("cuda:0")
    irr, n_nodes, n_edges, c, num_basis, r_max = "0e+1o+2e", 4096, 65536, 64, 8, 3.0

    class Layer(torch.nn.Module):
        """``fused``: the last linear of the radial network (no bias) is evaluated inside the edge kernels
        (``edge_tensor_product_uu_radial``), so the (E, P, C) weight tensor and its gradient never exist; else it is a
        ``torch.nn.Linear`` as in code written for the reference."""

        def __init__(self, fused=False):
            super().__init__()
            self.fused = fused
            self.basis = enn.BesselBasis(r_max, num_basis, trainable=False)
            self.cutoff = enn.PolynomialCutoff(r_max)
            self.tp = enn.SO3Linear(irr, irr, irr, c, c, internal_weights=False, feature_mode="uu")
            self.hidden = torch.nn.Sequential(torch.nn.Linear(num_basis, 16), torch.nn.SiLU())
            self.last = torch.nn.Linear(16, self.tp.num_paths * c, bias=not fused)
            self.mix = enn.IrrepsLinear(irr, irr, c, c)
            self.gate_lin = enn.IrrepsLinear(irr, "0e+0e+0e", c, c)
            self.gate = enn.Gate(irr, activation=torch.nn.Sigmoid())
            self.norm = enn.LayerRMSNorm(irr, c)

        def forward(self, x, edge_vec, plan):
            r = edge_vec.norm(dim=-1)
            feat = self.hidden(self.basis(r) * self.cutoff(r)[:, None])
            if self.fused:
                msg = edge_tensor_product_uu_radial(x, edge_vec, feat, self.last.weight.t().reshape(16, self.tp.num_paths, c),
                                                    plan, self.tp.tp_info_forward, edge_vectors=True)
            else:
                msg = edge_tensor_product_uu_vectors(x, edge_vec, self.last(feat).view(-1, self.tp.num_paths, c), plan,
                                                     self.tp.tp_info_forward)
            h = self.mix(msg)
            return self.norm(self.gate(h, self.gate_lin(h)))

    g = torch.Generator().manual_seed(1)
    plan = EdgePlan(torch.randint(0, n_nodes, (n_edges,), generator=g).to(dev),
                    torch.randint(0, n_nodes, (n_edges,), generator=g).to(dev), n_nodes)
    x = torch.randn(n_nodes, 9, c, generator=g).to(dev).requires_grad_(True)
    ev = (torch.randn(n_edges, 3, generator=g) * 1.2).to(dev).requires_grad_(True)
    ct = torch.randn(n_nodes, 9, c, generator=g).to(dev)

    def wall(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    def measure(layer):
        """(eager ms, replayed-graph ms, largest relative difference between a replay and an eager step)"""
        wrt = [x, ev] + list(layer.parameters())

        def step():
            return torch.autograd.grad(layer(x, ev, plan), wrt, ct)

        eager = wall(step)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            recorded = step()
        replay = wall(graph.replay)
        expect = step()
        torch.cuda.synchronize()
        err = max(float((a - b).abs().max() / b.abs().max().clamp_min(1e-30)) for a, b in zip(recorded, expect))
        return eager, replay, err

    torch.manual_seed(0)
    eager_ms, graph_ms, err = measure(Layer().to(dev))
    torch.manual_seed(0)
    fused_eager_ms, fused_graph_ms, fused_err = measure(Layer(fused=True).to(dev))
    print(json.dumps({"metric": "message-passing layer fwd+bwd Medges/s (lmax=2, C=64, fp32)",
                      "value": round(n_edges / (graph_ms * 1e-3) / 1e6, 1), "unit": "Medges/s", "n_gpus": 1,
                      "steps": steps, "warmup": warmup, "ms_per_step": round(graph_ms, 4), "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"layer: {n_nodes} nodes, {n_edges} edges, {irr}, {c} channels, "
                                             "one recorded HIP graph per step"},
                      "eager_ms_per_step": round(eager_ms, 4), "graph_ms_per_step": round(graph_ms, 4),
                      "graph_vs_eager_max_rel_err": err,
                      "last_radial_linear_in_the_edge_kernels": {
                          "eager_ms_per_step": round(fused_eager_ms, 4), "graph_ms_per_step": round(fused_graph_ms, 4),
                          "Medges_per_s": round(n_edges / (fused_graph_ms * 1e-3) / 1e6, 1),
                          "graph_vs_eager_max_rel_err": fused_err}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="edge_fwd_bwd", choices=sorted(WORKLOADS))
    ap.add_argument("--rotate", type=int, default=4, help="number of weight buffers cycled through")
    ap.add_argument("--graph", default="uniform", choices=["uniform", "local"],
                    help="edge workloads: uniform random src/dst (BASELINE) or edges between nearby node ids")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload: skip the compact records of the other BASELINE configurations")
    ap.add_argument("--cpu-sample-edges", type=int, default=16384)
    ap.add_argument("--pos-per-wave", type=int, default=0,
                    help="sorted positions per wavefront in the per-kernel timing (0 = library default)")
    ap.add_argument("--kernel-reps", type=int, default=100, help="launches per kernel for the roofline timing")
    ap.add_argument("--no-measure-traffic", action="store_true",
                    help="edge workloads: take roofline.traffic from the committed profile summary instead of measuring "
                         "it now with four short child runs under rocprofv3 --pmc (10-20 s)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no multi-GPU part); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    if args.workload in ("copy", "read"):
        membench(args.workload, args.steps, args.warmup)
        return
    if args.workload == "gemm":
        gemm_bench(args.steps, args.warmup)
        return
    if args.workload == "sh":
        sh_bench(args.steps, args.warmup)
        return
    if args.workload == "irreps_linear":
        irreps_linear_bench(args.steps, args.warmup)
        return
    if args.workload == "scatter":
        scatter_bench(args.steps, args.warmup)
        return
    if args.workload == "modules":
        modules_bench(args.steps, args.warmup)
        return
    if args.workload == "layer":
        layer_bench(args.steps, args.warmup)
        return
    if args.workload in ("uvw_fwd", "uvw_fwd_bwd"):
        print(json.dumps(uvw_bench(args)))
        return
    if args.workload == "edge_l6_fwd_bwd":
        print(json.dumps(edge_rows_bench(args)))
        return
    if args.workload in ("u1v_fp32_fwd_bwd", "uvw_fp32_fwd_bwd"):
        print(json.dumps(fp32_fully_connected_bench(args)))
        return
    if args.workload == "u1v_per_sample_fwd_bwd":
        print(json.dumps(per_sample_bench(args)))
        return
    if args.workload == "edge_table_fwd_bwd":
        print(json.dumps(edge_table_bench(args)))
        return
    if args.workload == "edge_radial_fwd_bwd":
        r = radial_record(16)
        print(json.dumps({
            "metric": "edge-TP fwd+bwd Medges/s (lmax=2,C=64, weights formed in the kernels, R=16)",
            "value": r["Medges_s"], "unit": "Medges/s", "n_gpus": 1, "steps": 20, "warmup": 3,
            "ms_per_step": r["step_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "edge_radial_fwd_bwd: N=4096 nodes, E=65536 edges, irreps 0e+1o+2e, C=64, "
                                   "h (E,16), W_last (16,11,64)"}, "kernels": r}))
        return

    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels

    lmax, ch, n_nodes, n_edges = WORKLOADS[args.workload]
    backward = args.workload == "edge_fwd_bwd"
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(dev)
    p = mod.num_paths
    inp = make_inputs(lmax, ch, n_nodes, n_edges, args.rotate, dev, args.graph)
    d = inp["d"]
    plan = EdgePlan(inp["src"].to(dev), inp["dst"].to(dev), n_nodes)
    x = inp["x"].to(dev).requires_grad_(backward)
    sh = inp["sh"].to(dev).requires_grad_(backward)
    ws = [torch.randn(n_edges, p, ch, generator=inp["gen"]).to(dev).requires_grad_(backward)
          for _ in range(args.rotate)]
    ct = torch.randn(n_nodes, d, ch, generator=inp["gen"]).to(dev)

    def step(i):
        w = ws[i % args.rotate]
        out = edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward)
        if backward:
            gx, gsh, gw = torch.autograd.grad(out, (x, sh, w), ct)
            return gw
        return out

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    # Host time to issue a step, over the first steps only: once the launch queue is full the host waits for the GPU
    # and its time per step reads the same as the GPU's.
    n_host = min(args.steps, 100)
    t0 = time.perf_counter()
    for i in range(args.steps):
        if i == n_host:
            host_elapsed = time.perf_counter() - t0
        step(i)
    if n_host == args.steps:
        host_elapsed = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    medges = n_edges / (elapsed / args.steps) / 1e6

    # ---- per-kernel durations with events on the launch stream (torch's current stream) ----------------------
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    xd, shd = x.detach(), sh.detach()

    def time_kernel(fn):
        """(average, median) launch duration in ms.  Average: one pair of events around all launches, issued back
        to back as in the step loop (a pair per launch adds the events' own ~1 us to every launch); median: of
        launches bracketed one by one."""
        wd = [w.detach() for w in ws]
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(args.kernel_reps):
            fn(wd[i % args.rotate])
        b.record()
        evs = []
        for i in range(args.kernel_reps):
            c, d_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            c.record()
            fn(wd[i % args.rotate])
            d_.record()
            evs.append((c, d_))
        torch.cuda.synchronize()
        ts = sorted(c.elapsed_time(d_) for c, d_ in evs)
        return a.elapsed_time(b) / args.kernel_reps, ts[len(ts) // 2]

    ppw = args.pos_per_wave
    fwd_fn = lambda w: kernels.uvu_forward(cfg, dims, xd, shd, w, seg=plan.fwd_index, pos_per_wave=ppw)
    bwd_fn = lambda w: kernels.uvu_backward(cfg, dims, xd, shd, w, ct, (True, True, True), seg=plan.bwd_index,
                                            pos_per_wave=ppw)
    fwd_fn(ws[0].detach()); bwd_fn(ws[0].detach())
    fwd_avg, fwd_med = time_kernel(fwd_fn)
    bwd_avg, bwd_med = time_kernel(bwd_fn)
    fwd_bytes, bwd_bytes = algorithmic_bytes(n_nodes, n_edges, d, p, ch)
    if backward:
        dom, dom_bytes, dom_ms = "cgtp::uvu_seg_bwd_kernel<TP_sh2,float,4,1>", bwd_bytes, bwd_avg
    else:
        dom, dom_bytes, dom_ms = "cgtp::uvu_seg_fwd_kernel<TP_sh2,float,4>", fwd_bytes, fwd_avg
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic, traffic_source = profiled_traffic(args.workload) if args.graph == "uniform" else (None, "not profiled")
    # measured now unless told otherwise, or unless this process itself runs under a profiler (its children would be
    # profiled twice)
    profiled = any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ) or "rocprof" in os.environ.get("LD_PRELOAD", "")
    traffic_measured = False
    if not args.no_measure_traffic and not profiled and args.graph == "uniform":
        live, live_source = measured_traffic(args.workload)
        if live is not None:
            traffic, traffic_source, traffic_measured = live, live_source, True
        else:
            traffic_source += f" (live measurement unavailable: {live_source})"
    # what this box itself delivers for plain streaming kernels, next to the vendor peak: the denominators a tuned
    # bandwidth-bound kernel can actually be held against
    copy_gbs, _ = stream_rate("copy", 10, 3)
    read_gbs, _ = stream_rate("read", 10, 3)

    rec = {
        "metric": "edge-TP fwd+bwd Medges/s (lmax=2,C=64)" if backward else "edge-TP fwd Medges/s (lmax=2,C=64)",
        "value": round(medges, 2), "unit": "Medges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "host_issue_ms_per_step": round(host_elapsed / n_host * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: N={n_nodes} nodes, E={n_edges} edges, irreps {irreps}, "
                               f"C={ch}, per-edge weights (E,{p},{ch}), {args.rotate} rotating weight buffers"
                               + ("" if args.graph == "uniform" else f", {args.graph} graph")},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_source, "traffic_measured": traffic_measured,
                     "algorithmic_bytes": dom_bytes, "avg_ms": round(dom_ms, 5),
                     "achievable": {"copy_GBs": round(copy_gbs, 1), "read_GBs": round(read_gbs, 1),
                                    "what": "1 GiB streaming copy (read + write bytes) and read kernels, same run",
                                    "frac_of_copy": round(achieved / copy_gbs, 4),
                                    "frac_of_read": round(achieved / read_gbs, 4),
                                    "traffic_GBs": None if traffic is None else round(traffic / dom_ms / 1e6, 1)}},
        "kernels": {"fwd_avg_ms": round(fwd_avg, 5), "fwd_med_ms": round(fwd_med, 5),
                    "fwd_GBs": round(fwd_bytes / fwd_avg / 1e6, 1),
                    "bwd_avg_ms": round(bwd_avg, 5), "bwd_med_ms": round(bwd_med, 5),
                    "bwd_GBs": round(bwd_bytes / bwd_avg / 1e6, 1),
                    "fwd_bwd_GBs": round((fwd_bytes + bwd_bytes) / (fwd_avg + bwd_avg) / 1e6, 1)},
    }
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(inp, lmax, ch, n_nodes, min(args.cpu_sample_edges, n_edges))
    if args.workload == "edge_fwd_bwd" and not args.no_configs and args.graph == "uniform":
        del x, sh, ws, ct, plan
        torch.cuda.empty_cache()
        rec["configs"] = other_configs(args, rec)
    print(json.dumps(rec))


def other_configs(args, headline):
    """Compact records of the other BASELINE configurations, timed in the same run with a few steps each so that the
    default command covers all five: [0] the CPU-reference module (B = 1024, C = 16, shared weight) on the oracle's
    CPU path and on the GPU; [1] the edge forward; [3] the bf16 fully connected product; [4] the lmax = 6 edge step."""
    import copy
    out = {}
    k = headline["kernels"]
    out["cfg1_edge_fwd_lmax2_C64"] = {"kernel_ms": k["fwd_avg_ms"], "GBs": k["fwd_GBs"],
                                      "hbm_frac": round(k["fwd_GBs"] / HBM_PEAK_GBS, 4),
                                      "Medges_s": round(65536 / (k["fwd_avg_ms"] * 1e-3) / 1e6, 1)}
    out["cfg0_uvu_B1024_C16_shared_w"] = config0_record(not args.no_cpu_baseline)
    sub = copy.copy(args)
    sub.steps, sub.warmup, sub.kernel_reps, sub.no_cpu_baseline = 50, 10, 30, True
    sub.workload = "uvw_fwd_bwd"
    r = uvw_bench(sub)
    flops = r["roofline"]["algorithmic_flops"]
    out["cfg3_uvw_bf16_B32768_C128"] = {
        "step_ms": r["ms_per_step"], "step_TFLOPs": r["value"], "step_mfma_frac": round(r["value"] / MFMA_BF16_PEAK_TFLOPS, 4),
        "fwd_ms": r["kernels"]["fwd_ms"], "fwd_TFLOPs": round(flops / (r["kernels"]["fwd_ms"] * 1e-3) / 1e12, 1),
        "fwd_mfma_frac": round(flops / (r["kernels"]["fwd_ms"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "grad_x_ms": r["kernels"]["grad_x_ms"], "grad_sh_ms": r["kernels"]["grad_sh_ms"],
        "grad_w_ms": r["kernels"]["grad_w_ms"]}
    torch.cuda.empty_cache()
    sub.workload, sub.steps, sub.warmup = "edge_l6_fwd_bwd", 20, 4
    r = edge_rows_bench(sub)
    torch.cuda.empty_cache()
    out["cfg1_edge_weights_formed_in_kernel_R16"] = radial_record(16)
    out["cfg4_edge_fwd_bwd_lmax6_C32"] = {
        "Medges_s": r["value"], "step_ms": r["ms_per_step"], "fwd_ms": r["kernels"]["fwd_ms"],
        "bwd_ms": r["kernels"]["bwd_ms"], "bwd_hbm_frac": r["roofline"]["frac"],
        "bwd_fp32_frac": r["roofline"]["fp32_vector"]["frac"],
        "bwd_fp32_frac_of_unpacked": r["roofline"]["fp32_vector"]["frac_of_unpacked"],
        "fwd_TFLOPs": r["kernels"]["fwd_TFLOPs"],
        "fwd_fp32_frac_of_unpacked": r["kernels"]["fwd_fp32_frac_of_unpacked"]}
    torch.cuda.empty_cache()
    # beside the BASELINE configurations: a weight per sample on the streaming kernels, and an edge step for irreps
    # without a compiled table on the fused table-driven kernels
    sub.workload, sub.steps, sub.warmup, sub.kernel_reps = "u1v_per_sample_fwd_bwd", 20, 3, 20
    r = per_sample_bench(sub)
    out["u1v_per_sample_weight_N65536_C16"] = {
        "step_ms": r["ms_per_step"], "Msamples_s": r["value"], "fwd_ms": r["kernels"]["fwd_ms"],
        "fwd_hbm_frac": r["kernels"]["fwd_frac_of_peak"], "fwd_frac_of_read_rate": r["kernels"]["fwd_frac_of_read"],
        "bwd_ms": r["kernels"]["bwd_ms"], "bwd_hbm_frac": r["roofline"]["frac"],
        "bwd_frac_of_copy_rate": r["roofline"]["achievable"]["frac_of_copy"]}
    torch.cuda.empty_cache()
    sub.workload, sub.kernel_reps = "edge_table_fwd_bwd", 10
    r = edge_table_bench(sub)
    out["edge_fwd_bwd_irreps_without_compiled_table"] = {
        "Medges_s": r["value"], "step_ms": r["ms_per_step"], "separate_launches_step_ms": r["kernels"]["separate"]["step_ms"],
        "per_coefficient_vs_compiled": r["kernels"]["per_coefficient_vs_compiled"]}
    torch.cuda.empty_cache()
    return out


FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X fp32 matrix, vendor figure


def fp32_fully_connected_bench(args):
    """``SO3Linear('uv')`` (u1v) or ``TensorProduct('uvw')`` with a shared fp32 weight, forward + backward through the
    public autograd API, and every kernel of the step on its own.  Algorithmic flops per product: 2 * B * S * K * C_out
    (S (path, output row) segments, K contracted channels; the coupling is not counted); the step has four."""
    from equitorch_amd.nn import SO3Linear, TensorProduct
    from equitorch_amd.nn.functional import _uv_native
    from equitorch_amd.utils._sh import spherical_harmonics
    lmax, ch, n = WORKLOADS[args.workload]
    uvw = args.workload.startswith("uvw")
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    d = (lmax + 1) ** 2
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, d, ch, generator=gen).to(dev)
    ct = torch.randn(n, d, ch, generator=gen).to(dev)
    if uvw:
        mod = TensorProduct(irreps, irreps, irreps, ch, ch, ch, feature_mode="uvw", internal_weights=False).to(dev)
        y = torch.randn(n, d, ch, generator=gen).to(dev)
        w = (torch.randn(mod.num_paths, ch, ch, ch, generator=gen) / ch).to(dev)
        k = ch * ch
    else:
        mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(dev)
        vec = torch.randn(n, 3, generator=gen)
        y = spherical_harmonics(vec / vec.norm(dim=-1, keepdim=True), lmax).to(dev)
        w = (torch.randn(mod.num_paths, ch, ch, generator=gen) / (ch * mod.num_paths) ** 0.5).to(dev)
        k = ch
    info = mod.tp_info_forward
    s1 = int(info.info_Mij_fwd.out_size)
    flops = 2.0 * n * s1 * k * ch
    xg, yg, wg = (t.clone().requires_grad_(True) for t in (x, y, w))

    def step():
        return torch.autograd.grad(mod(xg, yg, wg), (xg, yg, wg), ct)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3

    def timed(fn):
        evs = []
        for _ in range(args.kernel_reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(); b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs[2:]) / (len(evs) - 2)
    p = mod.num_paths
    if uvw:
        wp = _uv_native.pack(w, p, k, ch, k * ch, ch, 1)
        wt1 = w.permute(0, 2, 3, 1).contiguous()
        wp1 = _uv_native.pack(wt1, p, k, ch, k * ch, ch, 1)
        wt2 = w.permute(0, 3, 1, 2).contiguous()
        wp2 = _uv_native.pack(wt2, p, k, ch, k * ch, ch, 1)
        kern = {
            "fwd_ms": timed(lambda: _uv_native.apply(x, y, wp, info, "out", d, ch)),
            "grad_x_ms": timed(lambda: _uv_native.apply(y, ct, wp1, info, "in1_uvw", d, ch)),
            "grad_y_ms": timed(lambda: _uv_native.apply(ct, x, wp2, info, "in2_uvw", d, ch)),
            "grad_w_ms": timed(lambda: _uv_native.grad_w(x, y, ct, info)),
        }
    else:
        wp = _uv_native.pack(w, p, ch, ch, ch * ch, ch, 1)
        wpt = _uv_native.pack(w, p, ch, ch, ch * ch, 1, ch)
        kern = {
            "fwd_ms": timed(lambda: _uv_native.apply(x, y, wp, info, "out", d, ch)),
            "grad_x_ms": timed(lambda: _uv_native.apply(ct, y, wpt, info, "in1", d, ch)),
            "grad_y_ms": timed(lambda: _uv_native.grad_y(x, ct, wp, info, d)),
            "grad_w_ms": timed(lambda: _uv_native.grad_w(x, y, ct, info)),
        }
    tf = {key: flops / (v * 1e-3) / 1e12 for key, v in kern.items()}
    name = "uvw" if uvw else "u1v"
    return {
        "metric": f"{name} fp32 fwd+bwd TFLOP/s (lmax={lmax},C={ch})", "value": round(4 * flops / (ms_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: B={n}, irreps {irreps}, channels {ch}, shared weight {tuple(w.shape)}, "
                               f"forward + backward through the module"},
        "roofline": {"bound": "mfma", "kernel": "cgtp::uvt_apply_kernel (forward)", "achieved": round(tf["fwd_ms"], 2),
                     "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf["fwd_ms"] / FP32_MFMA_PEAK_TFLOPS, 4),
                     "traffic": None, "algorithmic_flops": flops, "avg_ms": round(kern["fwd_ms"], 5)},
        "kernels": {**{key: round(v, 5) for key, v in kern.items()},
                    **{key.replace("_ms", "_mfma_frac"): round(v / FP32_MFMA_PEAK_TFLOPS, 4) for key, v in tf.items()}}}


def _events_ms(fn, reps):
    """Average duration of ``fn`` from one pair of events around ``reps`` back-to-back calls on the current stream."""
    for _ in range(3):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def per_sample_bench(args):
    """``tensor_product_u1v`` with a weight per sample (N, P, C, C), fp32, forward + backward through autograd on the
    streaming kernels.  HBM-bound: the weight is read once forward; backward it is read once and its gradient written
    once.  Algorithmic bytes: N * P * C * C * 4 per pass over the weight (operands and output are 2-10 % more and are
    not counted).  The weight tensors rotate over two buffers (1.5 GB: past the last-level cache)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    lmax, ch, n = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    infos = [t.to(dev) for t in tp_infos(Irreps(irreps), Irreps(irreps), Irreps(irreps))[:3]]
    d, p = (lmax + 1) ** 2, kernels.coo_of(infos[0]).P
    gen = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(n, d, ch, device=dev, generator=gen).requires_grad_(True)
    y = torch.randn(n, d, device=dev, generator=gen).requires_grad_(True)
    ws = [torch.randn(n, p, ch, ch, device=dev, generator=gen).requires_grad_(True) for _ in range(2)]
    ct = torch.randn(n, d, ch, device=dev, generator=gen)
    w_bytes = ws[0].numel() * 4
    seen = []
    log, kernels.log_tier = kernels.log_tier, lambda op, tier, detail="": seen.append(tier)
    F.tensor_product_u1v(x, y, ws[0], *infos)
    kernels.log_tier = log
    if not seen or "streaming" not in seen[-1]:
        raise RuntimeError(f"the per-sample product did not take the streaming kernels: {seen}")
    count = [0]

    def fwd():
        count[0] += 1
        return F.tensor_product_u1v(x, y, ws[count[0] % 2], *infos)

    def step():
        out = fwd()
        torch.autograd.grad(out, (x, y, ws[count[0] % 2]), ct)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3
    with torch.no_grad():
        fwd_ms = _events_ms(fwd, args.kernel_reps)
    outs = [F.tensor_product_u1v(x, y, w, *infos) for w in ws]

    def bwd():
        count[0] += 1
        i = count[0] % 2
        torch.autograd.grad(outs[i], (x, y, ws[i]), ct, retain_graph=True)
    bwd_ms = _events_ms(bwd, args.kernel_reps)
    rate = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    copy_gbs, read_gbs = stream_rate("copy", 20, 3)[0], stream_rate("read", 20, 3)[0]
    return {
        "metric": f"u1v per-sample weight fwd+bwd Msamples/s (lmax={lmax},C={ch})", "value": round(n / (ms_step * 1e-3) / 1e6, 2),
        "unit": "Msamples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: N={n}, irreps {irreps}, {ch} -> {ch} channels, weight {tuple(ws[0].shape)} "
                               f"per sample ({w_bytes / 1e6:.0f} MB), forward + backward through autograd"},
        "roofline": {"bound": "hbm", "kernel": "cgtp::psw_bwd_kernel<float,4,false>", "achieved": round(rate(2 * w_bytes, bwd_ms), 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(rate(2 * w_bytes, bwd_ms) / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": 2 * w_bytes, "avg_ms": round(bwd_ms, 5),
                     "achievable": {"copy_GBs": round(copy_gbs, 1), "read_GBs": round(read_gbs, 1),
                                    "frac_of_copy": round(rate(2 * w_bytes, bwd_ms) / copy_gbs, 4)}},
        "kernels": {"fwd_ms": round(fwd_ms, 5), "fwd_GBs": round(rate(w_bytes, fwd_ms), 1),
                    "fwd_frac_of_peak": round(rate(w_bytes, fwd_ms) / HBM_PEAK_GBS, 4),
                    "fwd_frac_of_read": round(rate(w_bytes, fwd_ms) / read_gbs, 4),
                    "bwd_ms": round(bwd_ms, 5), "bwd_GBs": round(rate(2 * w_bytes, bwd_ms), 1)}}


def edge_table_bench(args):
    """The edge step (gather, channel-wise product, segment sum; forward + backward) for an irreps triple without a
    compiled table, on the fused table-driven kernels, next to the three separate launches they replace and to the
    compiled lmax = 2 table on the same graph."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    _, ch, n_nodes, n_edges = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(0)
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    plan = EdgePlan(src.to(dev), dst.to(dev), n_nodes)
    triple = ("0e+1o+2e+3o", "1o+2e+3o", "0e+1o+2e")
    fused_table = kernels.uvu_table_of
    res, nnz = {}, {}
    for name, (io, i1, i2), table_of in (("table", triple, fused_table), ("separate", triple, lambda *a: None),
                                         ("compiled", ("0e+1o+2e",) * 3, fused_table)):
        kernels.uvu_table_of = table_of
        try:
            mod = SO3Linear(i1, i2, io, ch, ch, internal_weights=False, feature_mode="uu").to(dev)
            nnz[name] = int(kernels.coo_of(mod.tp_info_forward).coef.shape[0])
            x = torch.randn(n_nodes, Irreps(i1).dim, ch, device=dev, requires_grad=True)
            y = torch.randn(n_edges, Irreps(i2).dim, device=dev, requires_grad=True)
            w = torch.randn(n_edges, mod.num_paths, ch, device=dev, requires_grad=True)
            ct = torch.randn(n_nodes, Irreps(io).dim, ch, device=dev)

            def fwd():
                return edge_tensor_product_uu(x, y, w, plan, mod.tp_info_forward)

            def step():
                torch.autograd.grad(fwd(), (x, y, w), ct)
            with torch.no_grad():
                f = _events_ms(fwd, args.kernel_reps)
            res[name] = {"fwd_ms": round(f, 4), "step_ms": round(_events_ms(step, args.kernel_reps), 4)}
        finally:
            kernels.uvu_table_of = fused_table
    ms_step = res["table"]["step_ms"]
    per_coef = {k: v["step_ms"] / nnz[k] for k, v in res.items()}
    return {
        "metric": "edge-TP fwd+bwd Medges/s (irreps without a compiled table, C=64)", "value": round(n_edges / (ms_step * 1e-3) / 1e6, 2),
        "unit": "Medges/s", "n_gpus": 1, "steps": args.kernel_reps, "warmup": 3, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: N={n_nodes} nodes, E={n_edges} edges, {triple[0]} <- {triple[1]} x {triple[2]} "
                               f"({nnz['table']} coefficients), C={ch}, per-edge weights"},
        "kernels": {**res, "coefficients": nnz,
                    "per_coefficient_vs_compiled": round(per_coef["table"] / per_coef["compiled"], 2),
                    "fused_vs_separate": round(res["separate"]["step_ms"] / ms_step, 2)}}


def radial_record(r):
    """The headline edge workload with the per-edge weights formed inside the kernels from ``h (E, r)`` and a shared
    ``(r, 11, 64)`` matrix (``edge_tensor_product_uu_radial``), next to the same step with the weights formed by a
    matrix product and read back by the plain kernels.  Bytes per edge: compulsory traffic of the forward launch."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_radial
    from equitorch_amd.ops import kernels
    lmax, ch, n_nodes, n_edges = WORKLOADS["edge_fwd_bwd"]
    dev = torch.device("cuda:0")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(dev)
    inp = make_inputs(lmax, ch, n_nodes, n_edges, 1, dev)
    d, p, gen = inp["d"], mod.num_paths, inp["gen"]
    plan = EdgePlan(inp["src"].to(dev), inp["dst"].to(dev), n_nodes)
    x = inp["x"].to(dev).requires_grad_(True)
    sh = inp["sh"].to(dev).requires_grad_(True)
    hs = [torch.randn(n_edges, r, generator=gen).to(dev).requires_grad_(True) for _ in range(4)]
    wl = (torch.randn(r, p, ch, generator=gen) / r ** 0.5).to(dev).requires_grad_(True)
    ct = torch.randn(n_nodes, d, ch, generator=gen).to(dev)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)

    def wall(fn, steps=20, warm=3):
        for i in range(warm):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    def events(fn, reps=12):
        evs = []
        for i in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(i); b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs[2:]) / (reps - 2)

    def fused(i):
        out = edge_tensor_product_uu_radial(x, sh, hs[i % 4], wl, plan, mod.tp_info_forward)
        return torch.autograd.grad(out, (x, sh, hs[i % 4], wl), ct)

    def unfused(i):
        w = (hs[i % 4] @ wl.view(r, -1)).view(n_edges, p, ch)
        out = edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward)
        return torch.autograd.grad(out, (x, sh, hs[i % 4], wl), ct)
    xd, shd, wld = x.detach(), sh.detach(), wl.detach()
    fwd_ms = events(lambda i: kernels.uvu_radial_forward(cfg, dims, xd, shd, hs[i % 4].detach(), wld, plan.fwd_index))
    bwd_ms = events(lambda i: kernels.uvu_radial_backward(cfg, dims, xd, shd, hs[i % 4].detach(), wld, ct,
                                                          (True, True, True, True), plan.bwd_index))
    node = n_nodes * d * ch * 4
    idx = 2 * n_edges * 8 + (n_nodes + 1) * 8
    fwd_bytes = n_edges * r * 4 + r * p * ch * 4 + n_edges * d * 4 + 2 * node + idx
    plain_fwd_bytes, _ = algorithmic_bytes(n_nodes, n_edges, d, p, ch)
    step_fused, step_unfused = wall(fused), wall(unfused)
    return {"R": r, "fwd_ms": round(fwd_ms, 4), "bwd_all_grads_ms": round(bwd_ms, 4),
            "fwd_bytes_per_edge": round(fwd_bytes / n_edges, 1),
            "plain_fwd_bytes_per_edge": round(plain_fwd_bytes / n_edges, 1),
            "step_ms": round(step_fused, 4), "step_ms_weights_by_matrix_product": round(step_unfused, 4),
            "Medges_s": round(n_edges / (step_fused * 1e-3) / 1e6, 1)}


def config0_record(with_cpu):
    """BASELINE configs[0]: ``SO3Linear('0e+1o+2e' x3, 16, 16, feature_mode='uu')`` with a shared weight on B = 1024
    rows, forward + backward: the oracle's restatement of the reference CPU path (all host threads up to 16) next to
    the same step on the GPU (wall time per step through the public API, launch-bound at this size)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.utils._sh import spherical_harmonics
    from oracle import ref_ops, ref_tables
    irr, n, c = "0e+1o+2e", 1024, 16
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, 9, c, generator=gen)
    v = torch.randn(n, 3, generator=gen)
    sh = spherical_harmonics(v / v.norm(dim=-1, keepdim=True), 2)
    w = torch.randn(11, c, generator=gen)
    ct = torch.randn(n, 9, c, generator=gen)
    rec = {}
    dev = torch.device("cuda:0")
    mod = SO3Linear(irr, irr, irr, c, c, internal_weights=False, feature_mode="uu").to(dev)
    xd, shd, wd = (t.to(dev).requires_grad_(True) for t in (x, sh, w))
    ctd = ct.to(dev)

    def gstep():
        return torch.autograd.grad(mod(xd, shd, wd), (xd, shd, wd), ctd)
    for _ in range(5):
        gstep()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(50):
        gstep()
    torch.cuda.synchronize()
    rec["gpu_ms_per_step"] = round((time.perf_counter() - t0) / 50 * 1e3, 4)
    if with_cpu:
        threads = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(threads)
        fwd, b1, b2, _ = ref_tables.tp_infos(irr, irr, irr)
        fwd, b1, b2 = (ref_ops.tables_to_torch(t) for t in (fwd, b1, b2))

        def cstep():
            out, inter = ref_ops.cpu_u1u_forward(x, sh, w, fwd)
            return out, ref_ops.cpu_u1u_backward(ct, x, sh, w, inter, fwd, b1, b2)
        for _ in range(3):
            cstep()
        times = []
        for _ in range(20):
            t0 = time.perf_counter()
            cstep()
            times.append(time.perf_counter() - t0)
        rec["cpu_ms_per_step"] = round(sorted(times)[10] * 1e3, 3)
        rec["cpu"] = f"oracle ref_ops.cpu_u1u_forward/backward, median of 20, {threads} threads, {cpu_model()}"
    return rec


if __name__ == "__main__":
    main()
