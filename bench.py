#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A "step" is one conv2d forward + backward over one synthetic batch at the headline shape
(B=256, 64 -> 128 channels, 56x56, 3x3, stride 1, pad 1, f32):

    forward      x' = zero-bordered x ;  y  = sum over taps  W[tap] . shift(x', tap)      (Conv2D)
    filter grad  gy' = zero-bordered gy ; gW[tap] = sum_b gy'_b . shift(x'_b, tap)^T       (Conv2DFilterGrad)
    input grad   gx = sum over taps  W[tap]^T . shift(gy', tap)                             (Conv2DTranspose)

Each contraction is one implicit GEMM over the filter taps: the im2col columns the reference
materialises (conv2d.rs:25-112, conv2d_transpose.rs:148-151) are never written.  The
column-materialising kernels (im2col, the GEMMs over columns, col2im) serve the other geometries
and are timed in the per-kernel section.

Inputs are resident in HBM before the timed region.  Every kernel launch inside the timed steps
is bracketed by events on the launch stream, so the per-kernel figures and the roofline object
come from the same K steps as `value`.  The CPU baseline (the oracle's restatement of the
reference path with OpenBLAS, timed on this machine's host cores on a bounded sample of the same
workload) is reported beside it; it is a baseline, not a target.

Prints ONE JSON line on stdout.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E

# headline workload
B, C, K, H, W, KH, PAD, STRIDE, DIL = 256, 64, 128, 56, 56, 3, 1, 1, 1

# HBM bytes per launch at the headline shape come from the tracked counter summaries under profiles/:
# two rocprofv3 --pmc passes over this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled
# by what the same counter reads for the --pmc-calibration copy kernel in the same pass (1 GiB in, 1 GiB out).
# Each entry: summary file, then (kernel name, statistic) pairs whose scaled fetch + write are added up.
# pad_border_fast_kernel runs twice per step (x with 64 channels, gy with 128): min is the x call, max the gy call
# (the same launch zeroes the slack around the planes and rewrites the filter in tap order).
CALIBRATION_KERNEL = "ag::ew_vec_kernel<ag::ScaleF<false> >"
CALIBRATION_KIB = float(1 << 20)
_STEP, _POOL, _COLS = ("profiles/conv2d_fwd_bwd_c4_hbm_traffic.txt", "profiles/maxpool_c4_hbm_traffic.txt",
                       "profiles/conv2d_columns_c4_hbm_traffic.txt")
_RED, _ADAM, _EW = ("profiles/reductions_hbm_traffic.txt", "profiles/adam_2pow26_hbm_traffic.txt",
                    "profiles/elementwise_256x128x56x56_hbm_traffic.txt")
_DL = "ag::gemm_dl_kernel<%s>"   # the last template argument: 1 = implicit convolution over filter taps, 3 = ordinary product
PROFILE_TRAFFIC = {
    # the step (column-free)
    "gemm_fwd": (_STEP, [(_DL % "128, 256, 32, 64, 64, 3, true, false, 1", "avg"), (_DL % "128, 128, 32, 64, 64, 3, true, false, 1", "avg")]),
    "gemm_filter_grad": (_STEP, [(_DL % "128, 192, 32, 32, 96, 3, true, true, 3", "avg"), ("ag::splitk_fold_vec_kernel", "avg")]),
    "gemm_input_grad": (_STEP, [(_DL % "64, 128, 32, 32, 64, 3, true, false, 1", "avg")]),
    "fwd_prepare": (_STEP, [("ag::pad_border_fast_kernel", "min")]),
    "input_grad_prepare": (_STEP, [("ag::pad_border_fast_kernel", "max")]),
    # per-kernel section: pooling, and the column-materialising operators
    "maxpool_fwd": (_POOL, [("ag::maxpool_fwd_lds_kernel<3, 2>", "avg")]),
    "maxpool_bwd": (_POOL, [("ag::maxpool_bwd_s2_kernel<true, 3, 16, false>", "avg")]),
    "im2col": (_COLS, [("ag::im2col_same_kernel<3, 3, 1, 16>", "avg")]),
    "col2im": (_COLS, [("ag::col2im_same_kernel<3, 3, 1, 16>", "avg")]),
    "gemm_fwd_columns": (_COLS, [(_DL % "128, 256, 32, 64, 64, 3, true, false, 3", "avg"), (_DL % "128, 64, 32, 64, 32, 3, true, false, 3", "avg")]),
    "gemm_filter_grad_columns": (_COLS, [(_DL % "128, 192, 32, 32, 96, 3, true, true, 3", "avg"), ("ag::splitk_fold_vec_kernel", "avg")]),
    "gemm_input_grad_columns": (_COLS, [(_DL % "192, 128, 32, 96, 32, 3, false, false, 3", "avg")]),
    # reductions: fold_rows_kernel<64, true> serves the first stage of axes (0,2,3) and the mean over (2,3) (the same
    # traffic: the whole tensor once); fold_cols_groups_kernel is the small second stage of axes (0,2,3) (min) and the
    # whole of axis 0 (max)
    "sum_all_2^26": (_RED, [("ag::sum_stage1_kernel", "avg"), ("ag::sum_stage2_kernel", "avg")]),
    "reduce_sum_[256,128,56,56]_axes_0_2_3": (_RED, [("ag::fold_rows_kernel<64, true>", "avg"), ("ag::fold_cols_groups_kernel", "min")]),
    "reduce_sum_[256,128,56,56]_axis_0": (_RED, [("ag::fold_cols_groups_kernel", "max")]),
    "reduce_mean_[256,128,56,56]_axes_2_3": (_RED, [("ag::fold_rows_kernel<64, true>", "avg")]),
    # Adam: the same kernel and traffic whatever the placement of the arrays
    "adam_2^26": (_ADAM, [("ag::adam_kernel", "avg"), ("ag::adam_tick_kernel", "avg")]),
    "adam_2^26_operands_2MiB_aligned": (_ADAM, [("ag::adam_kernel", "avg"), ("ag::adam_tick_kernel", "avg")]),
    # elementwise glue
    "relu_[256,128,56,56]": (_EW, [("ag::ew_vec_kernel<ag::ReluF>", "avg")]),
    "relu_grad_[256,128,56,56]": (_EW, [("ag::ew_vec_kernel<ag::ReluGradF>", "avg")]),
    "add_bias_relu_[256,128,56,56]": (_EW, [("ag::ew_vec_kernel<ag::BroadcastF<2, unsigned int> >", "avg")]),
    "add_n_2x[256,128,56,56]": (_EW, [("ag::ew_vec_kernel<ag::AddNF>", "avg")]),
}
_profile_cache = {}
_profile_strict = True   # False under --only: the passes that produce the summaries cannot depend on them


def _profile_table(path):
    """{counter: {kernel: {"avg","min","max"}}} of one summary file (lines as rocpd_summary.py prints them)."""
    import re
    if path not in _profile_cache:
        table = {}
        pat = re.compile(r"^(FETCH_SIZE|WRITE_SIZE)\s+n=\s*\d+\s+avg=\s*([\d.]+)\s+min=\s*([\d.]+)\s+max=\s*([\d.]+)\s+(.*\S)\s*$")
        with open(os.path.join(ROOT, path)) as f:
            for line in f:
                m = pat.match(line)
                if m:
                    table.setdefault(m.group(1), {})[m.group(5)] = {"avg": float(m.group(2)), "min": float(m.group(3)),
                                                                    "max": float(m.group(4))}
        _profile_cache[path] = table
    return _profile_cache[path]


def profile_traffic(key):
    """(HBM bytes per launch, summary file) of one benchmark entry, from the tracked counter summary.
    Raises when the file or one of the kernel names the entry is made of is missing: a figure from kernels
    that no longer exist must not be reported."""
    path, parts = PROFILE_TRAFFIC[key]
    table = _profile_table(path)
    total = 0.0
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        rows = table.get(counter, {})
        if CALIBRATION_KERNEL not in rows:
            raise RuntimeError(f"{path}: no {counter} line of the calibration kernel {CALIBRATION_KERNEL}")
        factor = CALIBRATION_KIB / rows[CALIBRATION_KERNEL]["avg"]
        for kernel, stat in parts:
            if kernel not in rows:
                raise RuntimeError(f"{path}: no {counter} line of {kernel} (entry {key}): re-run the counter passes "
                                   f"the file names after changing which kernels an entry launches")
            total += rows[kernel][stat] * factor * 1024.0
    return total, path


def traffic_fields(key, ms=None):
    """JSON fields of one entry's measured HBM traffic (and, given its duration, the fraction of HBM peak)."""
    try:
        nbytes = profile_traffic(key)[0]
    except (RuntimeError, OSError):
        if _profile_strict:
            raise
        return {}
    out = {"traffic_bytes": round(nbytes)}
    if ms is not None:
        out["frac_hbm_of_traffic"] = round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)
    return out


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--batch", type=int, default=B, help="images per step (headline: 256)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-micro", action="store_true", help="skip the per-kernel microbenchmarks")
    ap.add_argument("--cpu-images", type=int, default=B, help="images per step of the CPU baseline (default: the whole batch)")
    ap.add_argument("--only", choices=("pool", "columns", "chain", "config1", "config2", "stride2", "config5", "config3", "reduce", "adam",
                                       "elementwise"),
                    help="run only one part of the per-kernel section (for profiler passes): the two pooling kernels, "
                         "the column-materialising convolution kernels, the steps of configuration 1 / 2 through the host "
                         "operator layer, the stride-2 variant of the headline, the dilated and transposed convolutions of "
                         "configuration 5, the dense products of configuration 3, the reductions, Adam, or the elementwise glue")
    ap.add_argument("--no-traffic", action="store_true",
                    help="leave the HBM-traffic fields out (for the profiler passes that produce the summaries those "
                         "fields are read from)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch one plain copy kernel (ag_scale_f32 by 1.0) over 2^28 floats, "
                         "so that a rocprofv3 --pmc run of this command holds a kernel of known traffic "
                         "(1 GiB read, 1 GiB written) to scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


class Timer:
    """Accumulates event-bracketed durations per kernel name on the current stream."""

    def __init__(self, torch):
        self.torch = torch
        self.pending = []
        self.enabled = False

    def run(self, name, fn):
        if not self.enabled:
            return fn()
        a = self.torch.cuda.Event(enable_timing=True)
        b = self.torch.cuda.Event(enable_timing=True)
        a.record()
        out = fn()
        b.record()
        self.pending.append((name, a, b))
        return out

    def totals(self):
        """Median duration per name over the timed steps."""
        self.torch.cuda.synchronize()
        per = {}
        for name, a, b in self.pending:
            per.setdefault(name, []).append(a.elapsed_time(b))
        return {k: sorted(v)[len(v) // 2] for k, v in per.items()}


WARM_MS = float(os.environ.get("AG_BENCH_WARM_MS", "40"))


def time_events(torch, fn, iters, warm=3, warm_ms=WARM_MS):
    """Median duration of `fn` over `iters` calls between event pairs, enqueued behind about `warm_ms` milliseconds of
    the same call back to back with no host wait in between: the GPU raises its clocks over tens of milliseconds of
    load, and a leg of a few short calls after an idle gap is otherwise timed part-way up that ramp."""
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(warm):
        fn()
    b.record()
    b.synchronize()
    per = max(a.elapsed_time(b) / warm, 1e-3)
    for _ in range(min(4000, int(warm_ms / per))):
        fn()
    evs = []
    for _ in range(iters):
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return ts[len(ts) // 2]


def cpu_baseline(images):
    """conv2d fwd+bwd of the oracle (reference restatement + OpenBLAS) on `images` images."""
    import numpy as np
    from oracle import pyoracle as orc

    orc.build()
    blas = orc.load_openblas()
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        cores = min(cores, int(env))
    rng = np.random.default_rng(1)
    x = rng.standard_normal((images, C, H, W), dtype=np.float32)
    s = np.sqrt(6.0 / K)
    w = rng.uniform(-s, s, (K, C, KH, KH)).astype(np.float32)
    gy = rng.standard_normal((images, K, H, W), dtype=np.float32)

    def step():
        # batch-parallel stages (rayon in the reference): one BLAS thread per image task
        orc.blas_set_threads(1)
        y, cols = orc.conv2d_fwd(x, w, PAD, STRIDE, DIL, threads=cores)
        gx = orc.conv2d_transpose(gy, w, PAD, STRIDE, DIL, out_hw=(H, W), threads=cores)
        # image-sequential filter gradient: parallelism only inside BLAS
        orc.blas_set_threads(cores)
        gw = orc.conv2d_filter_grad(cols, gy, w.shape)
        return y, gx, gw

    step()
    reps, t0 = 0, time.perf_counter()
    while True:
        step()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 8.0 or reps >= 20:
            break
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": round(images * reps / dt, 2), "unit": "images/s", "cores": cores, "kind": "port",
        "sample": f"{images} of {B} images per step of the same conv2d fwd+bwd workload, {reps} timed steps after one warm-up, "
                  f"{cores} threads on {model}; BLAS: {blas or 'none (built-in loops, not OpenBLAS)'}",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as entry
    entry.load_package()
    from rust_autograd_amd import capi, kernels as Kn

    capi.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    Bn = args.batch
    OH = Kn.conv_out_size(H, KH, PAD, STRIDE, DIL)
    P, CK = OH * OH, C * KH * KH

    global _profile_strict
    if args.only:
        _profile_strict = False
        g = torch.Generator(device=dev)
        g.manual_seed(99)
        if args.only == "pool":
            res = micro_pool(torch, Kn, capi, dev, g, iters=3, only=True)
        elif args.only == "columns":
            res = micro_columns(torch, Kn, capi, dev, g, iters=3)
        elif args.only in ("stride2", "config5"):
            res = other_conv_configs(torch, Kn, dev, g, which=args.only)
        elif args.only == "config3":
            res = micro_matmul(torch, Kn, dev, g)
        elif args.only == "reduce":
            res = micro_reduce(torch, Kn, dev, g, iters=3)
        elif args.only == "adam":
            res = micro_adam(torch, Kn, dev, g, iters=3)
        elif args.only == "elementwise":
            res = micro_elementwise(torch, Kn, dev, g, iters=3)
        else:
            res = graph_steps(which=args.only)
        if args.pmc_calibration:
            calibration_copy(torch, Kn, capi, dev)
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "kernels": res}))
        return

    g = torch.Generator(device=dev)
    g.manual_seed(1234)
    x = torch.randn(Bn, C, H, W, device=dev, generator=g)
    s = (6.0 / K) ** 0.5
    w = (torch.rand(K, C, KH, KH, device=dev, generator=g) * 2 - 1) * s
    gy = torch.randn(Bn, K, OH, OH, device=dev, generator=g)
    y = torch.empty(Bn, K, OH, OH, device=dev)
    gx = torch.empty(Bn, C, H, W, device=dev)
    gw = torch.empty(K, C, KH, KH, device=dev)
    L = capi.lib()
    st, ptr, chk = Kn._stream, Kn._ptr, capi.check
    T = Timer(torch)
    fgeom = (Bn, C, H, W, K, KH, KH, PAD, STRIDE, 1)                # forward / filter gradient
    igeom = (Bn, K, OH, OH, C, KH, KH, PAD, STRIDE, 1, H, W)        # input gradient
    n_xpad, n_gypad = L.ag_conv2d_nocols_scratch_floats(*fgeom), L.ag_conv_input_grad_scratch_floats(*igeom)
    assert n_xpad > 0 and n_gypad > 0, "the headline geometry takes the column-free path"
    xpad = torch.empty(n_xpad, device=dev)
    gypad = torch.empty(n_gypad, device=dev)
    ws = torch.empty(max(16, L.ag_conv2d_filter_grad_nocols_f32_workspace(*fgeom)), dtype=torch.uint8, device=dev)

    def step():
        # Conv2D forward: zero-bordered copy of x (kept for the filter gradient), then one implicit GEMM over the taps
        T.run("fwd_prepare", lambda: chk(L.ag_conv2d_nocols_prepare_f32(st(), ptr(x), ptr(w), ptr(xpad), *fgeom)))
        T.run("gemm_fwd", lambda: chk(L.ag_conv2d_nocols_gemm_f32(st(), ptr(xpad), ptr(y), *fgeom)))
        # zero-bordered copy of gy, shared by both gradients
        T.run("input_grad_prepare", lambda: chk(L.ag_conv_input_grad_prepare_f32(st(), ptr(gy), ptr(w), ptr(gypad), *igeom)))
        # Conv2DFilterGrad: GEMM over the flattened padded planes, summed over images
        T.run("gemm_filter_grad", lambda: chk(L.ag_conv2d_filter_grad_nocols_f32(st(), ptr(xpad), ptr(gypad), ptr(gw), *fgeom,
                                                                                 ptr(ws), ws.numel())))
        # Conv2DTranspose (the input gradient): implicit GEMM over the taps
        T.run("gemm_input_grad", lambda: chk(L.ag_conv_input_grad_gemm_f32(st(), ptr(gypad), ptr(gx), *igeom)))

    if args.pmc_calibration:
        calibration_copy(torch, Kn, capi, dev)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly `steps` steps, nothing but the step's own launches on the stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    # per-kernel durations: the same steps again with an event pair around every entry (the event
    # records cost a few microseconds each on the stream, so they stay out of the timed region)
    T.enabled = True
    for _ in range(args.steps):
        step()
    per = T.totals()

    gemm_flop = 2.0 * K * P * CK * Bn            # identical for the three contractions
    kernels = {}
    for name in ("gemm_fwd", "gemm_filter_grad", "gemm_input_grad"):
        tf = gemm_flop / (per[name] * 1e-3) / 1e12
        kernels[name] = {"ms": round(per[name], 4), "TFLOP/s": round(tf, 2), "frac_mfma": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)}
    # bordered copies: read the tensor once, write its padded planes once
    for name, nbytes in (("fwd_prepare", 4.0 * (x.numel() + n_xpad)), ("input_grad_prepare", 4.0 * (gy.numel() + n_gypad))):
        gbs = nbytes / (per[name] * 1e-3) / 1e9
        kernels[name] = {"ms": round(per[name], 4), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
    with_traffic = Bn == B and not args.no_traffic
    if with_traffic:
        for name in kernels:
            kernels[name]["traffic_bytes"] = round(profile_traffic(name)[0])
    gemm_ms = sum(per[n] for n in ("gemm_fwd", "gemm_filter_grad", "gemm_input_grad"))
    gemm_tf = 3 * gemm_flop / (gemm_ms * 1e-3) / 1e12
    dominant = max(("gemm_fwd", "gemm_filter_grad", "gemm_input_grad"), key=lambda n: per[n])
    dom_tf = gemm_flop / (per[dominant] * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dominant, "achieved": round(dom_tf, 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(dom_tf / FP32_MFMA_PEAK_TFLOPS, 4),
                "traffic": round(profile_traffic(dominant)[0]) if with_traffic else None,
                "traffic_source": profile_traffic(dominant)[1] if with_traffic else None,
                "gemm_phase_TFLOP/s": round(gemm_tf, 2),
                "gemm_phase_frac": round(gemm_tf / FP32_MFMA_PEAK_TFLOPS, 4)}

    if not args.no_micro:
        kernels.update(micro(torch, Kn, capi, dev))

    out = {
        "metric": "conv2d fwd+bwd images/sec (B256 64->128 @56x56, 3x3 f32)",
        "value": round(Bn / (ms_per_step * 1e-3), 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"C4 conv2d fwd+bwd: x [{Bn},{C},{H},{W}] N(0,1), w [{K},{C},{KH},{KH}] glorot-uniform, "
                               f"stride {STRIDE} pad {PAD}; forward, filter gradient and input gradient per step, each an implicit (column-free) GEMM over zero-bordered copies of x / gy"},
        "roofline": roofline, "kernels": kernels,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_images)
    print(json.dumps(out))


def calibration_copy(torch, Kn, capi, dev):
    """One plain copy kernel of known traffic: 2^28 floats read, 2^28 floats written."""
    src = torch.ones(1 << 28, device=dev)
    dst = torch.empty_like(src)
    capi.check(capi.lib().ag_scale_f32(Kn._stream(), Kn._ptr(src), 1.0, Kn._ptr(dst), src.numel()))
    torch.cuda.synchronize()


def micro(torch, Kn, capi, dev):
    """Per-kernel microbenchmarks at the shapes of the other configurations (median of 10)."""
    g = torch.Generator(device=dev)
    g.manual_seed(99)
    res = micro_pool(torch, Kn, capi, dev, g)
    res.update(micro_columns(torch, Kn, capi, dev, g))
    res.update(micro_rest(torch, Kn, capi, dev, g))
    return res


def micro_pool(torch, Kn, capi, dev, g, iters=10, only=False):
    res = {}
    # max_pool2d 3x3 stride 2 on the conv output [256,128,56,56], forward and argmax backward
    x = torch.randn(256, 128, 56, 56, device=dev, generator=g)
    n_out = 256 * 128 * 27 * 27
    by = 4.0 * (x.numel() + 2 * n_out)
    Lp = capi.lib()
    sp, pp, cp = Kn._stream, Kn._ptr, capi.check
    gx = torch.empty_like(x)
    # The arrays a pooling kernel streams side by side (y and argmax; gy and the tap bytes) have the same extent.
    # hipMalloc and torch's allocator place every large array on a 2 MiB boundary, which sends such streams to
    # the same DRAM banks at the same time; the host operator layer's arena starts its blocks a rotating multiple of
    # 4 KiB into their allocation instead.  That placement is the headline entry; the aligned one is timed next to it.
    for suffix, step in (("", 4096), ("_operands_2MiB_aligned", 0)):
        if only and not step:
            continue  # the counter passes profile one placement
        yb, ab, gb = (torch.randn(n_out + 4 * step, device=dev, generator=g) for _ in range(3))
        tb = torch.zeros(n_out + 16 * step, dtype=torch.uint8, device=dev)
        y, am, gy, il = yb[:n_out], ab[step:step + n_out], gb[3 * step:3 * step + n_out], tb[8 * step:8 * step + n_out]
        place = ("y, argmax, taps, gy start 0, 16, 32, 48 KiB past a 2 MiB boundary (the host layer's arena staggers its blocks)" if step
                 else "every operand starts on a 2 MiB boundary")
        fwd = lambda taps: cp(Lp.ag_maxpool2d_fwd_f32(sp(), pp(x), pp(y), pp(am), pp(taps) if taps is not None else None,
                                                      256, 128, 56, 56, 3, 0, 2))
        bwd = lambda: cp(Lp.ag_maxpool2d_bwd_f32(sp(), pp(gy), pp(am), pp(il), pp(gx), 256, 128, 56, 56, 3, 0, 2))
        ms = time_events(torch, lambda: fwd(il), iters)
        res["maxpool_fwd" + suffix] = {"ms": round(ms, 4), "GB/s": round(by / ms / 1e6, 1), "frac_hbm": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
                                       **(traffic_fields("maxpool_fwd", ms) if step else {}),
                                       "note": "also writes one tap byte per output (23.9 MB, not counted in GB/s): the exact selection "
                                               "that the backward needs above 2^24 elements; " + place}
        if not only and step:
            ms = time_events(torch, lambda: fwd(None), iters)
            res["maxpool_fwd_reference_outputs"] = {"ms": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
                                                    "frac_hbm": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                    "note": "y and the f32-encoded argmax only, the reference's two outputs; " + place}
        ms = time_events(torch, bwd, iters)
        res["maxpool_bwd" + suffix] = {"ms": round(ms, 4), "GB/s": round(by / ms / 1e6, 1), "frac_hbm": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
                                       **(traffic_fields("maxpool_bwd", ms) if step else {}), "note": place}
        if not only and step:
            # the same backward with the gradient of the ReLU in front of the pooling applied as it stores: one more
            # operand (the ReLU's input) is read
            bwd_relu = lambda: cp(Lp.ag_maxpool2d_bwd_relu_f32(sp(), pp(gy), pp(am), pp(il), pp(x), pp(gx), 256, 128, 56, 56, 3, 0, 2))
            ms = time_events(torch, bwd_relu, iters)
            byr = by + 4.0 * x.numel()
            res["maxpool_bwd_relu_grad"] = {"ms": round(ms, 4), "GB/s": round(byr / ms / 1e6, 1), "frac_hbm": round(byr / ms / 1e6 / HBM_PEAK_GBS, 4),
                                            "note": "MaxPool2DGrad and ReLUGrad in one pass (two passes: the backward above plus a "
                                                    "read-read-write pass over [256,128,56,56]); " + place}
        del yb, ab, gb, tb, y, am, gy, il
    return res


def micro_columns(torch, Kn, capi, dev, g, iters=10):
    res = {}
    # the column-materialising operators (what the reference does per image): im2col + W . cols, gy . cols^T summed
    # over images, W^T . gy + col2im
    Bn, Cc, Kf, Hh = 256, 64, 128, 56
    Pp, CKk = Hh * Hh, Cc * 9
    L = capi.lib()
    st, ptr, chk = Kn._stream, Kn._ptr, capi.check
    wt = torch.randn(Kf, CKk, device=dev, generator=g) * 0.1
    gyy = torch.randn(Bn, Kf, Pp, device=dev, generator=g)
    gc = torch.empty(Bn, CKk, Pp, device=dev)
    gxx = torch.empty(Bn, Cc, Hh, Hh, device=dev)
    xx = torch.randn(Bn, Cc, Hh, Hh, device=dev, generator=g)
    yy = torch.empty(Bn, Kf, Pp, device=dev)
    gww = torch.empty(Kf, CKk, device=dev)
    wsf = torch.empty(max(16, L.ag_conv2d_filter_grad_f32_workspace(Bn, CKk, Pp, Kf)), dtype=torch.uint8, device=dev)
    cb = 4.0 * (gc.numel() + gxx.numel())
    gf = 2.0 * Kf * Pp * CKk * Bn
    ms = time_events(torch, lambda: chk(L.ag_im2col_f32(st(), ptr(xx), ptr(gc), Bn, Cc, Hh, Hh, 3, 3, 1, 1, 1, 1, 1, 1)), iters)
    res["im2col"] = {"ms": round(ms, 4), "GB/s": round(cb / ms / 1e6, 1), "frac_hbm": round(cb / ms / 1e6 / HBM_PEAK_GBS, 4),
                     **traffic_fields("im2col")}
    ms = time_events(torch, lambda: chk(L.ag_gemm_f32(st(), 0, 0, Kf, Pp, CKk, 1.0, ptr(wt), CKk, 0, ptr(gc), Pp, CKk * Pp, 0.0,
                                                      ptr(yy), Pp, Kf * Pp, Bn)), iters)
    res["gemm_fwd_columns"] = {"ms": round(ms, 4), "TFLOP/s": round(gf / ms / 1e9, 2), "frac_mfma": round(gf / ms / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4),
                               **traffic_fields("gemm_fwd_columns")}
    ms = time_events(torch, lambda: chk(L.ag_gemm_batchsum_f32(st(), 0, 1, Kf, CKk, Pp, 1.0, ptr(gyy), Pp, Kf * Pp, ptr(gc), Pp,
                                                               CKk * Pp, 0.0, ptr(gww), CKk, Bn, ptr(wsf), wsf.numel())), iters)
    res["gemm_filter_grad_columns"] = {"ms": round(ms, 4), "TFLOP/s": round(gf / ms / 1e9, 2),
                                       "frac_mfma": round(gf / ms / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4),
                                       **traffic_fields("gemm_filter_grad_columns")}
    del xx, yy, gww, wsf
    ms = time_events(torch, lambda: chk(L.ag_gemm_f32(st(), 1, 0, CKk, Pp, Kf, 1.0, ptr(wt), CKk, 0, ptr(gyy), Pp, Kf * Pp,
                                                      0.0, ptr(gc), Pp, CKk * Pp, Bn)), iters)
    tf = 2.0 * Kf * Pp * CKk * Bn / ms / 1e9
    res["gemm_input_grad_columns"] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac_mfma": round(tf / FP32_MFMA_PEAK_TFLOPS, 4),
                                      **traffic_fields("gemm_input_grad_columns")}
    ms = time_events(torch, lambda: chk(L.ag_col2im_f32(st(), ptr(gc), ptr(gxx), Bn, Cc, Hh, Hh, 3, 3, 1, 1, 1, 1, 1, 1, Hh, Hh)), iters)
    res["col2im"] = {"ms": round(ms, 4), "GB/s": round(cb / ms / 1e6, 1), "frac_hbm": round(cb / ms / 1e6 / HBM_PEAK_GBS, 4),
                     **traffic_fields("col2im")}
    return res


def micro_rest(torch, Kn, capi, dev, g, iters=10):
    res = {}
    # a plain copy (ag_scale_f32 by 1.0) of 2^28 floats: what a streaming kernel with one read and one write stream reaches
    src = torch.ones(1 << 28, device=dev)
    dst = torch.empty_like(src)
    ms = time_events(torch, lambda: capi.check(capi.lib().ag_scale_f32(Kn._stream(), Kn._ptr(src), 1.0, Kn._ptr(dst), src.numel())), 10)
    res["copy_2^28"] = {"ms": round(ms, 4), "GB/s": round(8.0 * src.numel() / ms / 1e6, 1),
                        "frac_hbm": round(8.0 * src.numel() / ms / 1e6 / HBM_PEAK_GBS, 4)}
    del src, dst
    res.update(micro_reduce(torch, Kn, dev, g, iters))
    res.update(micro_adam(torch, Kn, dev, g, iters))
    res.update(micro_elementwise(torch, Kn, dev, g, iters))
    res.update(micro_matmul(torch, Kn, dev, g))
    res.update(other_conv_configs(torch, Kn, dev, g))
    res.update(graph_steps())
    return res


def hbm_entry(key, ms, nbytes, note=None):
    """One bandwidth-bound entry: algorithmic bytes over the measured time, plus the counter-derived traffic of the
    tracked summary where PROFILE_TRAFFIC names the entry."""
    e = {"ms": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    if key in PROFILE_TRAFFIC:
        e.update(traffic_fields(key, ms))
    if note:
        e["note"] = note
    return e


def micro_reduce(torch, Kn, dev, g, iters=10):
    """reduce_sum to a scalar on 2^26 elements and the axis reductions over the pool input's shape [256,128,56,56]:
    the per-channel (conv bias) gradient, one axis, the rows.  Algorithmic bytes: 4 per input element."""
    res = {}
    n = 1 << 26
    a = torch.randn(n, device=dev, generator=g)
    ms = time_events(torch, lambda: Kn.sum_all(a), iters)
    res["sum_all_2^26"] = hbm_entry("sum_all_2^26", ms, 4.0 * n)
    del a
    a4 = torch.randn(256, 128, 56, 56, device=dev, generator=g)
    for name, axes in (("reduce_sum_[256,128,56,56]_axes_0_2_3", [0, 2, 3]), ("reduce_sum_[256,128,56,56]_axis_0", [0]),
                       ("reduce_mean_[256,128,56,56]_axes_2_3", [2, 3])):
        fn = Kn.reduce_mean if "mean" in name else Kn.reduce_sum
        ms = time_events(torch, lambda: fn(a4, axes), iters)
        res[name] = hbm_entry(name, ms, 4.0 * a4.numel())
    return res


def micro_adam(torch, Kn, dev, g, iters=10):
    """The fused Adam update on 2^26 elements (28 bytes per element: p, g, m, v read; p, m, v written), with the four
    arrays 4 KiB apart modulo 2 MiB (what the host operator layer's arena hands out) and with all four on 2 MiB
    boundaries (what hipMalloc and torch's allocator hand out)."""
    res = {}
    n = 1 << 26
    a = torch.randn(n, device=dev, generator=g)
    t = torch.ones(1, device=dev)
    for name, step in (("adam_2^26", 1024), ("adam_2^26_operands_2MiB_aligned", 0)):
        bufs = [torch.zeros(n + 3 * step, device=dev) for _ in range(4)]
        ga, p, m, v = (b[i * step:i * step + n] for i, b in enumerate(bufs))
        ga.copy_(a)
        p.normal_(generator=g)
        ms = time_events(torch, lambda: Kn.adam_update(p, ga, m, v, t), iters)
        res[name] = hbm_entry(name, ms, 28.0 * n,
                              "param, grad, m, v start 0, 4, 8, 12 KiB past a 2 MiB boundary (the host layer's arena placement)"
                              if step else "param, grad, m, v all start on a 2 MiB boundary")
        del bufs, ga, p, m, v
    return res


def micro_elementwise(torch, Kn, dev, g, iters=10):
    """The elementwise glue at the headline activation shape [256,128,56,56] (411 MB per operand)."""
    res = {}
    x = torch.randn(256, 128, 56, 56, device=dev, generator=g)
    gy = torch.randn_like(x)
    bias = torch.randn(1, 128, 1, 1, device=dev, generator=g)
    nb = 4.0 * x.numel()
    ms = time_events(torch, lambda: Kn.relu(x), iters)
    res["relu_[256,128,56,56]"] = hbm_entry("relu_[256,128,56,56]", ms, 2 * nb)
    ms = time_events(torch, lambda: Kn.relu_grad(x, gy), iters)
    res["relu_grad_[256,128,56,56]"] = hbm_entry("relu_grad_[256,128,56,56]", ms, 3 * nb)
    ms = time_events(torch, lambda: Kn.add_broadcast_relu(x, bias), iters)
    res["add_bias_relu_[256,128,56,56]"] = hbm_entry("add_bias_relu_[256,128,56,56]", ms, 2 * nb,
                                                     "relu(x + b) with b [1,128,1,1] in one pass")
    ms = time_events(torch, lambda: Kn.add_n([x, gy]), iters)
    res["add_n_2x[256,128,56,56]"] = hbm_entry("add_n_2x[256,128,56,56]", ms, 3 * nb,
                                               "AddN of two gradients (also AddOp of equal shapes); the gradient of a [1,128,1,1] "
                                               "bias is the entry reduce_sum_[256,128,56,56]_axes_0_2_3")
    return res


def micro_matmul(torch, Kn, dev, g):
    """The dense contractions of configuration 3: 4096^3 in the three layouts of forward and gradients, 64 x 512^3."""
    res = {}
    A = torch.randn(4096, 4096, device=dev, generator=g)
    Bm = torch.randn(4096, 4096, device=dev, generator=g)
    for name, ta, tb in (("matmul_4096_NN", False, False), ("matmul_4096_NT", False, True), ("matmul_4096_TN", True, False)):
        ms = time_events(torch, lambda: Kn.matmul(A, Bm, ta, tb), 10, warm=10)
        tf = 2.0 * 4096 ** 3 / ms / 1e9
        res[name] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac_mfma": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)}
    del A, Bm
    A = torch.randn(64, 512, 512, device=dev, generator=g)
    Bm = torch.randn(64, 512, 512, device=dev, generator=g)
    for name, ta, tb in (("batch_matmul_64x512", False, False), ("batch_matmul_64x512_NT", False, True),
                         ("batch_matmul_64x512_TN", True, False)):
        ms = time_events(torch, lambda: Kn.batch_matmul(A, Bm, ta, tb), 10)
        tf = 2.0 * 64 * 512 ** 3 / ms / 1e9
        res[name] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac_mfma": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)}
    return res


def other_conv_configs(torch, Kn, dev, g, which=None):
    """Operator-level conv2d forward + both gradients at the remaining convolution configurations
    (stride-2 variant of the headline; dilated and transposed convolutions of configuration 5).  Each entry holds
    the time of the three operators launched back to back and of each operator on its own."""
    out = {}
    L = Kn.capi.lib()

    def entry(Bn, flop, ms_all, parts, path=None):
        e = {"ms": round(ms_all, 4), "images/s": round(Bn / ms_all * 1e3, 1), "TFLOP/s": round(flop / ms_all / 1e9, 2),
             "frac_mfma": round(flop / ms_all / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4)}
        for k, ms in parts.items():
            e[k + "_ms"] = round(ms, 4)
            e[k + "_frac_mfma"] = round(flop / 3 / ms / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4)
        if path:
            e["path"] = path
        return e

    def conv_case(name, Bn, Cc, Kf, Hh, k, pad, stride, dil):
        """Forward, filter gradient and input gradient the way the host Conv2D operator runs them:
        column-free where the library supports the geometry, over materialised columns otherwise."""
        x = torch.randn(Bn, Cc, Hh, Hh, device=dev, generator=g)
        w = torch.randn(Kf, Cc, k, k, device=dev, generator=g) * 0.05
        y, cols = Kn.conv2d(x, w, pad, stride, dil)
        gy = torch.randn_like(y)
        free = Kn.conv2d_nocols(x, w, pad, stride, dil) is not None and \
            Kn.conv_input_grad_staged(gy, w, pad, (Hh, Hh), stride, dil) is not None and \
            L.ag_conv2d_filter_grad_nocols_f32_workspace(Bn, Cc, Hh, Hh, Kf, k, k, pad, stride, dil) > 0
        if free:
            del cols
            yy, xp = Kn.conv2d_nocols(x, w, pad, stride, dil)
            gx, scratch = Kn.conv_input_grad_staged(gy, w, pad, (Hh, Hh), stride, dil)
            fwd = lambda: Kn.conv2d_nocols(x, w, pad, stride, dil)
            igrad = lambda: Kn.conv_input_grad_staged(gy, w, pad, (Hh, Hh), stride, dil)
            fgrad = lambda: Kn.conv2d_filter_grad_nocols(xp, scratch, tuple(x.shape), tuple(w.shape), pad, stride, dil)
        else:
            fwd = lambda: Kn.conv2d(x, w, pad, stride, dil)
            igrad = lambda: Kn.conv2d_transpose(gy, w, pad, stride, dil, out_hw=(Hh, Hh))
            fgrad = lambda: Kn.conv2d_filter_grad(cols, gy, tuple(w.shape))

        def step():
            fwd()
            igrad()     # (its bordered copy of gy is what the column-free filter gradient reads)
            fgrad()

        ms = time_events(torch, step, 8)
        parts = {"fwd": time_events(torch, fwd, 8), "input_grad": time_events(torch, igrad, 8),
                 "filter_grad": time_events(torch, fgrad, 8)}
        flop = 3 * 2.0 * Bn * Kf * y.shape[2] * y.shape[3] * Cc * k * k
        out[name] = entry(Bn, flop, ms, parts, "column-free" if free else "columns")

    if which in (None, "stride2"):
        conv_case("conv2d_fwd_bwd_stride2_B256_64to128_56x56", 256, 64, 128, 56, 3, 1, 2, 1)
    if which in (None, "config5"):
        conv_case("conv2d_fwd_bwd_dilated_B32_256to256_14x14", 32, 256, 256, 14, 3, 2, 1, 2)
        # transposed convolution 128 -> 64, 4x4, stride 2, pad 1: [32,128,14,14] -> [32,64,28,28], forward and both gradients
        x = torch.randn(32, 128, 14, 14, device=dev, generator=g)
        w = (torch.rand(128, 64, 4, 4, device=dev, generator=g) - 0.5) * 0.2
        yt = Kn.conv2d_transpose(x, w, 1, 2)
        go = torch.randn_like(yt)
        fwd = lambda: Kn.conv2d_transpose(x, w, 1, 2)
        igrad = lambda: Kn.conv2d(go, w, 1, 2)                  # gradient w.r.t. the input of the transposed conv
        fgrad = lambda: Kn.conv2d_transpose_filter_grad(x, go, tuple(w.shape), 1, 2)

        def tstep():
            fwd()
            igrad()
            fgrad()

        ms = time_events(torch, tstep, 8)
        parts = {"fwd": time_events(torch, fwd, 8), "input_grad": time_events(torch, igrad, 8),
                 "filter_grad": time_events(torch, fgrad, 8)}
        tflop = 3 * 2.0 * 32 * 128 * 14 * 14 * 64 * 16
        out["conv2d_transpose_fwd_bwd_B32_128to64_14to28"] = entry(32, tflop, ms, parts)
    return out


def graph_steps(which=None):
    """Configurations 1 and 2 end to end through the host operator layer (graph build, evaluation,
    gradients, Adam), host arrays fed every step as the reference's examples do.  These steps are
    tens of MFLOP: launch- and copy-latency bound, reported as wall-clock time only."""
    import gc
    import time

    import numpy as np

    import rust_autograd_amd.graph as G

    rng = np.random.default_rng(5)

    def glorot(shape):
        sc = np.sqrt(6.0 / (int(np.prod(shape[1:])) + shape[0] * int(np.prod(shape[2:]))))
        return rng.uniform(-sc, sc, shape).astype(np.float32)

    out = {}
    # config 1: conv(1->32, 3x3, pad 1) -> ReLU -> max_pool 2x2 -> sum; grads w.r.t. x and w
    env = G.VariableEnvironment()
    wid = env.set("w", glorot((32, 1, 3, 3)))
    xv = rng.random((64, 1, 28, 28), dtype=np.float32)

    def c1_step():
        c = env.context()
        x, w = c.placeholder("x", [-1, 1, 28, 28]), c.variable(wid)
        loss = c.reduce_sum(c.max_pool2d(c.relu(c.conv2d(x, w, 1, 1)), 2, 0, 2), [0, 1, 2, 3])
        c.eval(c.grad([loss], [x, w]), {"x": xv})

    # config 2: the small CNN of examples/cnn_mnist.rs with Adam, batch 128
    env2 = G.VariableEnvironment()
    params = {"w1": glorot((32, 1, 3, 3)), "w2": glorot((64, 32, 3, 3)),
              "w3": rng.uniform(-0.04, 0.04, (3136, 10)).astype(np.float32),
              "b1": np.zeros((1, 32, 28, 28), np.float32), "b2": np.zeros((1, 64, 14, 14), np.float32),
              "b3": np.zeros((1, 10), np.float32)}
    ids = {k: env2.set(k, a) for k, a in params.items()}
    names = list(params)
    adam = G.Adam(env2, [ids[k] for k in names], alpha=1e-3)
    x2 = rng.random((128, 1, 28, 28), dtype=np.float32)
    y2 = rng.integers(0, 10, (128, 1)).astype(np.float32)

    def c2_step():
        c = env2.context()
        v = {k: c.variable(ids[k]) for k in names}
        x, t = c.placeholder("x", [-1, 1, 28, 28]), c.placeholder("y", [-1, 1])
        z = c.max_pool2d(c.relu(c.conv2d(x, v["w1"], 1, 1) + v["b1"]), 2, 0, 2)
        z = c.max_pool2d(c.relu(c.conv2d(z, v["w2"], 1, 1) + v["b2"]), 2, 0, 2)
        logits = c.matmul(c.reshape(z, [-1, 3136]), v["w3"]) + v["b3"]
        loss = c.reduce_mean(c.sparse_softmax_cross_entropy(logits, t), [0], False)
        grads = c.grad([loss], [v[k] for k in names])
        adam.update([v[k] for k in names], grads, c, {"x": x2, "y": y2})

    if which in (None, "chain"):
        out.update(chain_step(G, np, rng, glorot, time, gc))
    for name, step, images in (("config1_conv_block_step", c1_step, 64), ("config2_cnn_adam_step", c2_step, 128)):
        if which is not None and not name.startswith(which):
            continue
        for _ in range(50):   # (the arena reaches its working size and the clocks their sustained level)
            step()
        G.synchronize()
        # Wall clock of 200 consecutive steps, device idle before and after.  A config-1 step reads its two
        # gradients back, so it ends with the device idle; a config-2 step (Optimizer::update) returns once its
        # work is enqueued, and the host builds the next graph while the device runs the step.
        n_steps = 200
        # (the interpreter's cyclic collector is held off as timeit does: its first full pass over everything torch's
        # import created takes about 36 ms, once, and would land in the timed region)
        gc.collect()
        gc.disable()
        try:
            t0 = time.perf_counter()
            for _ in range(n_steps):
                step()
            G.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / n_steps
        finally:
            gc.enable()
        out[name] = {"ms": round(ms, 3), "images/s": round(images / ms * 1e3, 1),
                     "note": "graph build + host feeds + evaluation through libag_host.so, wall clock per step over 200 consecutive steps after 50 warm-up steps"}
    return out


def chain_step(G, np, rng, glorot, time, gc):
    """conv(64->128, 3x3) -> ReLU -> max_pool 2x2 -> conv(128->128, 3x3) at the headline's input [256,64,56,56], forward and
    the gradients w.r.t. the input and both filters, through the host operator layer with everything resident on the
    device -- once with the evaluator's shortcuts (the ReLU inside the pooling's launch, one bordered copy of gy for both
    gradients of a convolution) and once node by node."""
    env = G.VariableEnvironment()
    xid = env.set("x", rng.standard_normal((256, 64, 56, 56), dtype=np.float32))
    w1, w2 = env.set("w1", glorot((128, 64, 3, 3))), env.set("w2", glorot((128, 128, 3, 3)))
    flop = 3 * 2.0 * 256 * 128 * 576 * 56 * 56 + 3 * 2.0 * 256 * 128 * 1152 * 28 * 28

    def step():
        c = env.context()
        x, a, b = c.variable(xid), c.variable(w1), c.variable(w2)
        y = c.conv2d(c.max_pool2d(c.relu(c.conv2d(x, a, 1, 1)), 2, 0, 2), b, 1, 1)
        gx, ga, gb = c.grad([c.reduce_sum(y, [0, 1, 2, 3])], [x, a, b])
        c.eval([c.reduce_sum(gx, [0, 1, 2, 3]), ga, gb])   # (the input gradient is summed so that 205 MB need not come back)

    res = {}
    for key, on in (("", True), ("_node_by_node", False)):
        G.set_shortcuts(on)
        try:
            for _ in range(5):
                step()
            G.synchronize()
            gc.collect()
            gc.disable()
            try:
                t0 = time.perf_counter()
                for _ in range(20):
                    step()
                G.synchronize()
                ms = (time.perf_counter() - t0) * 1e3 / 20
            finally:
                gc.enable()
        finally:
            G.set_shortcuts(True)
        res["ms" + key] = round(ms, 3)
    ms = res["ms"]
    return {"chain_conv_relu_pool_conv_B256_56x56": {
        **res, "images/s": round(256 / ms * 1e3, 1), "TFLOP/s": round(flop / ms / 1e9, 2),
        "frac_mfma": round(flop / ms / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4),
        "note": "graph build + evaluation through libag_host.so of conv(64->128) -> ReLU -> max_pool 2x2 -> conv(128->128), forward and "
                "gradients w.r.t. input and filters (0.533 TFLOP of contractions), wall clock per step over 20 steps; ms_node_by_node: "
                "the same with the evaluator's shortcuts off (every node on its own, a bordered copy of gy per gradient)"}}


if __name__ == "__main__":
    main()
