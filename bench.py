#!/usr/bin/env python3
"""Benchmark of the conv2d_gw8 hot path on one MI355X.

Workloads (--workload):
  target, cfg1, cfg2, cfg3   one convolution shape.  A step is one pass of the hot path over one
             batch of synthetic input: the forward kernel, then the backward half as the
             product's backward op runs it (one fused data+weight gradient kernel where the
             recorded times say it is faster, else the data-gradient and weight-gradient
             kernels), including the zero fill of grad_weight.  Everything is launched through
             the C ABI on torch's current stream with every tensor resident in HBM; launches
             rotate over buffer sets that together exceed the 256 MB memory-side cache several
             times, so the rates are HBM rates.
  cfg4       forward (and backward) at C=64 56x56 3x3 for batch sizes 1..512.
  cfg5       inference of a ConvNeXt-Tiny-shaped network with gw8 convolutions at batch 128.
The default run (target) also carries a `configs` block: compact measurements of cfg1, cfg2, cfg3
(per-kernel us, fraction of the HBM roofline, counter traffic), the cfg4 batch sweep and cfg5 (the
four convolution and LayerNorm shapes and the network's ms per iteration); --no-configs leaves it out.

The single JSON line printed at the end reports
  value      effective GB/s of the whole step = the algorithmic bytes the launched kernels move
             (a fused backward kernel reads grad_output once and is counted once) / step time;
             `reference_accounting` prices the same time with the reference's three-direction
             byte count (scripts/plot_kernel_bench.py:430-435),
  kernels    per-kernel us (median and min over repeated event-timed blocks), effective GB/s and
             fraction of the 8 TB/s roofline,
  roofline   the same for the kernel that takes the most time, with the HBM traffic and the MFMA
             utilisation measured by rocprofv3 counters when a summary for this workload is in
             profiles/ (`traffic_stale` / `mfma_util_stale`: the kernel source has changed since),
  copy_ceiling  the best of a few tuned streaming copies of the same volume (what HBM gives a
             read-X/write-X kernel on this device), and the plain copy beside it,
  torch_gpu_conv2d  torch's own grouped conv2d (MIOpen) on the same GPU and shapes,
  cpu_baseline  the reference's CPU oracle path (torch conv2d fp32, groups=C/8, and its
             autograd) on the host cores for a bounded sample, all threads and one thread.

The timed region is `--steps` steps between synchronisations, repeated until at least 0.2 s have
been measured; ms_per_step is the median block, so the sample size does not depend on --steps.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]
"""

import argparse
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
# the run-time compiler's thread pool: the benchmark compiles some sixty kernels (read at import)
os.environ.setdefault("SPIO_WORKERS", str(max(4, min(16, (os.cpu_count() or 4)))))

HBM_PEAK_GBS = 8000.0
CACHE_BYTES = 256 * 1024 * 1024
MIN_TIMED_SECONDS = 0.2
METRIC = "conv2d_gw8 effective HBM bandwidth (fwd+dgrad+wgrad step)"

WORKLOADS = {
    # name: (description, params kwargs, weight seed)
    "target": ("conv2d_gw8 fwd+dgrad+wgrad N=128 C=64 56x56 3x3 pad1 fp16 NHWC",
               dict(n=128, c=64, h=56, w=56, padding=1, r=3, s=3), 0),
    "cfg1": ("conv2d_gw8 fwd+dgrad+wgrad N=32 C=64 56x56 3x3 pad1 fp16 NHWC",
             dict(n=32, c=64, h=56, w=56, padding=1, r=3, s=3), 0),
    "cfg2": ("conv2d_gw8 fwd+dgrad+wgrad N=128 C=128 28x28 3x3 pad1 fp16 NHWC",
             dict(n=128, c=128, h=28, w=28, padding=1, r=3, s=3), 1),
    "cfg3": ("conv2d_gw8 fwd+dgrad+wgrad N=256 C=256 14x14 7x7 pad3 fp16 NHWC",
             dict(n=256, c=256, h=14, w=14, padding=3, r=7, s=7), 2),
}  # fmt: skip
SWEEP_BATCHES = (1, 2, 4, 8, 16, 32, 64, 128, 256, 512)
NETWORK_WIDTHS = ((96, 56), (192, 28), (384, 14), (768, 7))
LAUNCH_FLOOR_US = 2.2  # an empty kernel in the same back-to-back loop
WARM_SECONDS = 0.03  # of back-to-back launches before a kernel is timed
# What a plain streaming kernel needs for a given volume on this device: the launch floor plus the
# bytes at the marginal rate of the copy kernels (their time against size is a fixed 1.5-2.4 us
# plus 6.0-6.4 TB/s).  `frac_of_stream_model` = that time / the kernel's: a kernel near 1 has
# nothing left but the launch floor and the bytes, whatever its share of the 8 TB/s peak is.
STREAM_RATE_GBS = 6200.0


def stream_model(us, nbytes):
    model = LAUNCH_FLOOR_US + nbytes / (STREAM_RATE_GBS * 1e3)
    return {"stream_model_us": round(model, 2), "frac_of_stream_model": round(model / us, 3)}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="target", choices=sorted(WORKLOADS) + ["cfg4", "cfg5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-torch-gpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-batch", type=int, default=32)
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload only: leave out the compact cfg1-cfg5 block")
    return ap.parse_args()


# ------------------------------------------------------------------ helpers


def source_digest(source_file):
    """Short hash of a kernel source and the header it includes: what a counter figure in
    profiles/ was measured with."""
    import hashlib

    h = hashlib.sha256()
    for name in (source_file, "spio_conv_common.h"):
        try:
            with open(os.path.join(ROOT, "spio_amd", "csrc", name), "rb") as f:
                h.update(f.read())
        except OSError:
            return None
    return h.hexdigest()[:12]


def profile_figure(kind, workload, kernel, source_file=None):
    """A per-launch figure from the rocprofv3 counter summaries in profiles/: (value, stale).

    The summaries carry lines `<kind> <workload> <kernel> <value> [<source file>:<digest>]` with
    kind `traffic_bytes` (FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the same
    counter reads for the plain copy kernel) or `mfma_util` (per cent of the cycles in which the
    matrix pipes were busy, the profiler's MfmaUtil).  `stale` is True when the line names the
    digest of the kernel source it was measured with and today's source differs, None when it
    names none.  (None, None) without a summary."""
    pdir = os.path.join(ROOT, "profiles")
    try:
        names = sorted(os.listdir(pdir))
    except OSError:
        return None, None
    pat = re.compile(rf"{kind}\s+{re.escape(workload)}\s+{re.escape(kernel)}\s+([0-9.]+)(?:\s+(\S+):([0-9a-f]+))?")
    for name in names:
        try:
            with open(os.path.join(pdir, name), "r", encoding="utf-8") as f:
                m = pat.search(f.read())
        except OSError:
            continue
        if m:
            value = float(m.group(1)) if kind == "mfma_util" else int(float(m.group(1)))
            stale = None
            if m.group(3):
                stale = source_digest(m.group(2)) != m.group(3)
            return value, stale
    return None, None


def attach_profile_figures(entry, workload, name):
    """Adds traffic / mfma_util (and their stale flags) from profiles/ to a kernel entry."""
    entry["traffic"], stale = profile_figure("traffic_bytes", workload, name)
    if stale is not None:
        entry["traffic_stale"] = stale
    util, ustale = profile_figure("mfma_util", workload, name)
    if util is not None:
        entry["mfma_util"] = round(util / 100.0, 4)
        if ustale is not None:
            entry["mfma_util_stale"] = ustale


def rotation_sets(set_bytes):
    """Buffer sets so that one pass over all of them touches >= 4x the memory-side cache."""
    return max(2, min(16, -(-4 * CACHE_BYTES // max(set_bytes, 1))))


def timed_blocks(run_block, min_seconds=MIN_TIMED_SECONDS, max_blocks=400):
    """Repeat `run_block()` (which returns the seconds it took) until min_seconds have been
    measured; returns the list of block times."""
    times = []
    total = 0.0
    while (total < min_seconds or len(times) < 3) and len(times) < max_blocks:
        t = run_block()
        times.append(t)
        total += t
    return times


def time_kernel(kernel, arg_sets, iters, min_seconds=MIN_TIMED_SECONDS):
    """Median and min microseconds per call over repeated event-timed blocks of `iters` launches."""
    # warm-up: the first tens of milliseconds after a pause (new buffers, another kernel's set-up)
    # read up to 5 % slow
    warm = 0.0
    while warm < WARM_SECONDS:
        warm += kernel.time(arg_sets, warmup=10, iters=iters) * 1e-3 * iters
    per_call = []
    total = 0.0
    while (total < min_seconds or len(per_call) < 3) and len(per_call) < 400:
        ms = kernel.time(arg_sets, warmup=0, iters=iters)
        per_call.append(ms * 1e3)
        total += ms * 1e-3 * iters
    return statistics.median(per_call), min(per_call), len(per_call)


def kernel_entry(kernel, arg_sets, nbytes, iters, min_seconds=MIN_TIMED_SECONDS):
    med, mn, blocks = time_kernel(kernel, arg_sets, iters, min_seconds)
    gbs = nbytes / (med * 1e-6) / 1e9
    return {
        "us": round(med, 2),
        "us_min": round(mn, 2),
        "blocks": blocks,
        "bytes": nbytes,
        "GB/s": round(gbs, 1),
        "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
        "config": dict(vars(kernel.config)),
        "kernel": kernel.kernel_name,
        "source": kernel.kernel_source_file,
        "source_digest": source_digest(kernel.kernel_source_file),
    }


def make_buffers(params, seed, nsets, device):
    """nsets independent (x, dy, y, dx, dw) sets plus the shared weights."""
    import torch

    cl = torch.channels_last
    gen = torch.Generator().manual_seed(seed)
    fan_in = 8 * params.r * params.s
    bound = (6.0 / (6.0 * fan_in)) ** 0.5  # kaiming_uniform_(a=sqrt(5)), the nn.Conv2d default
    w = ((torch.rand(params.weight_shape, generator=gen) * 2 - 1) * bound).half()
    w = w.to(device).contiguous(memory_format=cl)
    sets = []
    for i in range(nsets):
        g = torch.Generator(device=device).manual_seed(1000 + i)
        x = torch.randn(params.input_shape, device=device, dtype=torch.float16, generator=g)
        dy = torch.randn(params.output_shape, device=device, dtype=torch.float16, generator=g)
        sets.append(dict(
            x=x.contiguous(memory_format=cl),
            dy=dy.contiguous(memory_format=cl),
            y=torch.empty(params.output_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl),
            dx=torch.empty(params.input_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl),
            dw=torch.zeros(params.weight_shape, device=device, dtype=torch.float32).contiguous(memory_format=cl),
        ))  # fmt: skip
    return w, sets


def copy_ceiling(nbytes, device, iters):
    """What HBM gives a kernel that reads `nbytes` and writes `nbytes`: the plain one-load-one-store
    copy and a few tuned grid-stride variants (independent loads in flight per lane, workgroup
    size, grid as a multiple of the CU count); the best is the ceiling."""
    import torch

    from spio_amd.compiler.compile_kernel import compile_and_load_kernel
    from spio_amd.hip import get_device_attributes

    cus = get_device_attributes(device.index or 0).multiprocessor_count
    n = nbytes // 16
    nsets = rotation_sets(2 * nbytes)
    sets = []
    for _ in range(nsets):
        src = torch.randint(0, 2**31 - 1, (n * 4,), dtype=torch.int32, device=device)
        sets.append((torch.empty_like(src), src))
    stream = torch.cuda.current_stream(device).cuda_stream

    def run(fn, grid, threads, args_of):
        asets = [args_of(d, s) for d, s in sets]
        fn.launch_timed((grid, 1, 1), (threads, 1, 1), asets, 0, stream, 10, iters)
        per_call, total = [], 0.0
        while (total < MIN_TIMED_SECONDS / 2 or len(per_call) < 3) and len(per_call) < 200:
            ms = fn.launch_timed((grid, 1, 1), (threads, 1, 1), asets, 0, stream, 0, iters)
            per_call.append(ms * 1e3)
            total += ms * 1e-3 * iters
        return statistics.median(per_call)

    variants = []
    _m0, plain = compile_and_load_kernel("spio_stream_copy", "stream_copy.hip", {}, device.index or 0)
    us = run(plain, (n + 255) // 256, 256, lambda d, s: (d, s, n))
    variants.append({"kernel": "spio_stream_copy", "threads": 256, "unroll": 1, "grid": (n + 255) // 256,
                     "us": round(us, 2), "GB/s": round(2 * n * 16 / us / 1e3, 1)})  # fmt: skip
    keep = [_m0]
    for threads, unroll, mult in ((512, 1, 16), (256, 2, 16), (256, 4, 8), (1024, 1, 8), (512, 2, 4), (256, 8, 4)):
        chunks = n // (threads * unroll)
        if chunks == 0:
            continue
        grid = min(chunks, cus * mult)
        defines = {"SPIO_COPY_THREADS": threads, "SPIO_COPY_UNROLL": unroll}
        m, fn = compile_and_load_kernel("spio_stream_copy_strided", "stream_copy.hip", defines, device.index or 0)
        keep.append(m)
        us = run(fn, grid, threads, lambda d, s, g=grid: (d, s, n, g))
        variants.append({"kernel": "spio_stream_copy_strided", "threads": threads, "unroll": unroll,
                         "grid": grid, "us": round(us, 2), "GB/s": round(2 * n * 16 / us / 1e3, 1)})  # fmt: skip
    # two tensors in, one out: the fused backward kernel's mix (every set gets a second source of
    # its own, so that no launch reads what its predecessor has just read)
    second = {id(s): torch.randint(0, 2**31 - 1, (n * 4,), dtype=torch.int32, device=device) for _d, s in sets}
    combine = []
    for threads, unroll, mult in ((512, 1, 16), (256, 2, 16), (256, 4, 8), (512, 2, 8)):
        chunks = n // (threads * unroll)
        if chunks == 0:
            continue
        grid = min(chunks, cus * mult)
        defines = {"SPIO_COPY_THREADS": threads, "SPIO_COPY_UNROLL": unroll}
        m, fn = compile_and_load_kernel("spio_stream_combine_strided", "stream_copy.hip", defines, device.index or 0)
        keep.append(m)
        us = run(fn, grid, threads, lambda d, s, g=grid: (d, s, second[id(s)], n, g))
        combine.append({"kernel": "spio_stream_combine_strided", "threads": threads, "unroll": unroll,
                        "grid": grid, "us": round(us, 2), "GB/s": round(3 * n * 16 / us / 1e3, 1)})  # fmt: skip
    del sets, second
    best = max(variants, key=lambda v: v["GB/s"])
    best2 = max(combine, key=lambda v: v["GB/s"]) if combine else None
    return {
        "bytes": 2 * n * 16,
        "buffer_sets": nsets,
        "best": best,
        "plain": variants[0],
        "frac_of_hbm_peak": round(best["GB/s"] / HBM_PEAK_GBS, 4),
        "variants": variants,
        "two_in_one_out": {"bytes": 3 * n * 16, "best": best2, "variants": combine,
                           "note": "dst = a ^ b over three tensors of the same size: the HBM rate a kernel that "
                                   "reads two activation tensors and writes one reaches (the fused backward's mix)"},
        "note": "non-temporal copies of one activation tensor in and one out over rotating buffers: "
                "the HBM rate a read-X/write-X kernel reaches on this device",
    }


def torch_gpu_conv2d(params, sets, w, iters):
    """The framework's own grouped conv2d on the same GPU (MIOpen through torch), fp16
    channels_last, same shapes: the comparison the reference draws against PyTorch/cuDNN
    (figures/batch_size_vs_eff_bandwidth__*.png).  torch.cuda events on the current stream."""
    import torch
    import torch.nn.functional as F

    pad = (params.padding_h, params.padding_w)
    out = {}
    try:
        x0 = sets[0]["x"].detach().requires_grad_(True)
        w0 = w.detach().requires_grad_(True)
        y0 = F.conv2d(x0, w0, None, 1, pad, 1, params.groups)

        def fwd(i):
            F.conv2d(sets[i % len(sets)]["x"], w, None, 1, pad, 1, params.groups)

        def dgrad(i):
            torch.autograd.grad(y0, x0, sets[i % len(sets)]["dy"], retain_graph=True)

        def wgrad(i):
            torch.autograd.grad(y0, w0, sets[i % len(sets)]["dy"], retain_graph=True)

        for name, fn in (("fprop", fwd), ("dgrad", dgrad), ("wgrad", wgrad)):
            for i in range(3):
                fn(i)
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for i in range(iters):
                fn(i)
            stop.record()
            torch.cuda.synchronize()
            out[name + "_us"] = round(start.elapsed_time(stop) * 1e3 / iters, 2)
        out["note"] = ("torch.nn.functional.conv2d(groups=C/8) fp16 channels_last and its autograd on the "
                       "same GPU; dgrad/wgrad call torch.autograd.grad on one saved graph (input rotates only "
                       "for the upstream gradient)")
    except Exception as e:  # pylint: disable=broad-except
        out["error"] = f"{type(e).__name__}: {e}"[:200]
    return out


def physical_cores():
    """Distinct (package, core) pairs in /proc/cpuinfo, or None."""
    try:
        seen, phys, core = set(), None, None
        with open("/proc/cpuinfo", "r", encoding="utf-8") as f:
            for line in f:
                if line.startswith("physical id"):
                    phys = line.split(":")[1].strip()
                elif line.startswith("core id"):
                    core = line.split(":")[1].strip()
                elif not line.strip():
                    if phys is not None and core is not None:
                        seen.add((phys, core))
                    phys = core = None
        return len(seen) or None
    except OSError:
        return None


def cpu_baseline(params_kwargs, seed, sample_batch):
    """The reference's oracle path on the host cores, on a bounded sample of the workload:
    all threads (the `value`) and one thread."""
    import torch

    from oracle import conv2d_gw8_oracle as oracle
    from spio_amd.kernels import Conv2dGw8Params, Conv2dStats

    kw = dict(params_kwargs)
    kw["n"] = min(kw["n"], sample_batch)
    p = Conv2dGw8Params(**kw)
    x, w, _b, dy = oracle.make_args(p.n, p.c, p.h, p.w, p.r, p.s, p.padding_h, p.padding_w, False, seed)
    stats = Conv2dStats(p, output_names=["output", "grad_input", "grad_weight"])

    def one_pass():
        oracle.fprop_torch(x, w, None, p.padding_h, p.padding_w)
        oracle.grads_torch(x, w, None, dy, p.padding_h, p.padding_w)

    def measure(budget_s, min_runs, max_runs):
        one_pass()
        times = []
        t_end = time.perf_counter() + budget_s
        while len(times) < min_runs or (time.perf_counter() < t_end and len(times) < max_runs):
            t0 = time.perf_counter()
            one_pass()
            times.append(time.perf_counter() - t0)
        return statistics.median(times), len(times)

    threads = torch.get_num_threads()
    med, runs = measure(12.0, 5, 400)
    torch.set_num_threads(1)
    try:
        med1, runs1 = measure(8.0, 3, 100)
    finally:
        torch.set_num_threads(threads)
    return {
        "value": round(stats.bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": (
            f"torch.nn.functional.conv2d fp32 groups=C/8 forward + autograd grads (the function the "
            f"reference's tests use as oracle), batch {p.n} of {params_kwargs['n']} of the same "
            f"workload, median of {runs} passes, {med * 1e3:.1f} ms/pass on {threads} threads"
        ),
        "ms_per_pass": round(med * 1e3, 3),
        "single_thread": {"value": round(stats.bytes / med1 / 1e9, 3), "unit": "GB/s", "cores": 1,
                          "ms_per_pass": round(med1 * 1e3, 3), "passes": runs1},
        "logical_cpus": os.cpu_count(),
        "physical_cores": physical_cores(),
    }


# ------------------------------------------------------------------ workloads


def bench_conv(args, device, workload=None, full=True):
    """One convolution shape: the fwd + backward step, its kernels, the yardsticks.  `full=False`
    (the compact entries of the default run's `configs` block) leaves out the graph replay, the
    copy ceiling and the torch and CPU baselines, and times shorter blocks."""
    import torch

    from spio_amd.functional import fused_backward_kernel
    from spio_amd.kernels import (
        Conv2dGw8Params,
        Conv2dStats,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )

    workload = workload or args.workload
    min_seconds = MIN_TIMED_SECONDS if full else MIN_TIMED_SECONDS / 4
    desc, pkw, seed = WORKLOADS[workload]
    params = Conv2dGw8Params(**pkw)
    act_bytes = 2 * params.n * params.c * params.h * params.w
    out_bytes = 2 * params.n * params.c * params.p * params.q
    # the forward kernel alone touches x and y of a set: size the rotation for that
    nsets = rotation_sets(act_bytes + out_bytes)
    w, sets = make_buffers(params, seed, nsets, device)

    # First use: reads the recorded choice (or tunes), compiles and loads.
    t0 = time.perf_counter()
    k_fwd = conv2d_gw8_kernel_factory.get_kernel(params, device)
    k_dgrad = conv2d_gw8_kernel_factory.get_kernel(params, device, igrad=True)
    k_wgrad = conv2d_gw8_wgrad_kernel_factory.get_kernel(params, device)
    k_fused = fused_backward_kernel(params, device)
    setup_s = time.perf_counter() - t0

    def step(i):
        s = sets[i % nsets]
        k_fwd(s["y"], s["x"], w, None)
        s["dw"].zero_()
        if k_fused is not None:
            k_fused(s["dx"], s["dw"], s["x"], s["dy"], w)
        else:
            k_dgrad(s["dx"], s["dy"], w, None)
            k_wgrad(s["dw"], s["x"], s["dy"])

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    def block():
        t = time.perf_counter()
        for i in range(args.steps):
            step(i)
        torch.cuda.synchronize()
        return time.perf_counter() - t

    blocks = timed_blocks(block, min_seconds)
    ms_per_step = statistics.median(blocks) * 1e3 / args.steps
    ms_per_step_min = min(blocks) * 1e3 / args.steps

    # The same steps replayed from HIP graphs (one graph per buffer set): what a caller that
    # captures its training step gets; reported beside the eager figure, which stays `value`.
    graph_ms_per_step = long_graph_ms_per_step = None
    try:
        if not full:
            raise _Skip()
        graphs = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(nsets):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    step(i)
                graphs.append(g)
        torch.cuda.current_stream().wait_stream(side)
        for i in range(args.warmup):
            graphs[i % nsets].replay()
        torch.cuda.synchronize()

        def gblock():
            t = time.perf_counter()
            for i in range(args.steps):
                graphs[i % nsets].replay()
            torch.cuda.synchronize()
            return time.perf_counter() - t

        graph_ms_per_step = statistics.median(timed_blocks(gblock)) * 1e3 / args.steps
        del graphs
        # ... and one graph that holds a step for every buffer set: a replay then submits
        # 3 * nsets kernels at once, so what a graph launch itself costs is spread over them
        long_graph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(long_graph, stream=side):
                for i in range(nsets):
                    step(i)
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(3):
            long_graph.replay()
        torch.cuda.synchronize()
        replays = max(1, args.steps // nsets)

        def lblock():
            t = time.perf_counter()
            for _ in range(replays):
                long_graph.replay()
            torch.cuda.synchronize()
            return time.perf_counter() - t

        long_graph_ms_per_step = statistics.median(timed_blocks(lblock)) * 1e3 / (replays * nsets)
        del long_graph
    except _Skip:
        pass
    except Exception as e:  # pylint: disable=broad-except
        print(f"bench.py: HIP graph replay skipped: {type(e).__name__}: {e}", file=sys.stderr)

    # Per-kernel times with HIP events on the launch stream.
    iters = max(20, min(args.steps, 200))
    st = {
        "fprop": Conv2dStats(params, output_names="output"),
        "dgrad": Conv2dStats(params, output_names="grad_input"),
        "wgrad": Conv2dStats(params, output_names="grad_weight"),
    }
    nbytes = {
        "fprop": st["fprop"].bytes,
        "dgrad": st["dgrad"].bytes,
        # grad_weight is fp32 on the device
        "wgrad": st["wgrad"].bytes_read + st["wgrad"].grad_weight_bytes_written_fp32,
    }
    nbytes["bgrad"] = nbytes["dgrad"] + nbytes["wgrad"] - out_bytes  # grad_output is read once
    kernels = {
        "fprop": kernel_entry(k_fwd, [(s["y"], s["x"], w, None) for s in sets], nbytes["fprop"], iters, min_seconds),
        "dgrad": kernel_entry(k_dgrad, [(s["dx"], s["dy"], w, None) for s in sets], nbytes["dgrad"], iters, min_seconds),
        "wgrad": kernel_entry(k_wgrad, [(s["dw"], s["x"], s["dy"]) for s in sets], nbytes["wgrad"], iters, min_seconds),
    }
    if k_fused is not None:
        kernels["bgrad"] = kernel_entry(
            k_fused, [(s["dx"], s["dw"], s["x"], s["dy"], w) for s in sets], nbytes["bgrad"], iters, min_seconds
        )
        kernels["bgrad"]["note"] = ("fused dgrad+wgrad as the backward op runs it for this shape; replaces "
                                    "the dgrad and wgrad launches in the timed step")
        ref_bytes = nbytes["dgrad"] + nbytes["wgrad"]
        kernels["bgrad"]["reference_accounting"] = {
            "bytes": ref_bytes,
            "GB/s": round(ref_bytes / (kernels["bgrad"]["us"] * 1e-6) / 1e9, 1),
            "note": "the same time priced with the bytes the two separate kernels need for this work",
        }

    in_step = ["fprop", "bgrad"] if k_fused is not None else ["fprop", "dgrad", "wgrad"]
    step_bytes = sum(nbytes[n] for n in in_step)  # what the timed step moves
    ref_step_bytes = nbytes["fprop"] + nbytes["dgrad"] + nbytes["wgrad"]
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    dominant = max(in_step, key=lambda n: kernels[n]["us"])
    for name in kernels:
        attach_profile_figures(kernels[name], workload, name)
        # what an empty kernel costs in the same back-to-back loop, as a share of this kernel's time
        kernels[name]["launch_floor_share"] = round(LAUNCH_FLOOR_US / kernels[name]["us"], 3)
        kernels[name].update(stream_model(kernels[name]["us"], kernels[name]["bytes"]))
    roofline = {
        "bound": "hbm",
        "kernel": kernels[dominant]["kernel"],
        "achieved": kernels[dominant]["GB/s"],
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": kernels[dominant]["frac_of_hbm_peak"],
        "traffic": kernels[dominant]["traffic"],
    }
    for key in ("traffic_stale", "mfma_util", "mfma_util_stale"):
        if key in kernels[dominant]:
            roofline[key] = kernels[dominant][key]
    if not full:
        del sets
        torch.cuda.empty_cache()
        compact = {}
        for name, e in kernels.items():
            compact[name] = {k: e[k] for k in ("us", "us_min", "GB/s", "frac_of_hbm_peak", "traffic", "traffic_stale",
                                               "mfma_util", "launch_floor_share", "frac_of_stream_model", "bytes") if k in e}
            compact[name]["config"] = {k: v for k, v in e["config"].items() if v not in (0, None)}
        return {
            "workload": desc, "params": params.encode(), "step_kernels": in_step,
            "step_us": round(ms_per_step * 1e3, 2), "step_GB/s": round(value, 1),
            "step_frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4), "step_bytes": step_bytes,
            "first_use_seconds": round(setup_s, 2), "buffer_sets": nsets, "kernels": compact,
            "roofline": roofline,
        }  # fmt: skip

    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": desc,
            "params": params.encode(),
            "buffer_sets": nsets,
            "first_use_seconds": round(setup_s, 2),
            "step_kernels": in_step,
        },
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "value_note": "algorithmic bytes of the kernels the step launches (" + " + ".join(in_step)
                      + ") divided by the median time of one step",
        "timed_blocks": len(blocks),
        "ms_per_step_min": round(ms_per_step_min, 5),
        "step_bytes": step_bytes,
        "reference_accounting": {
            "bytes": ref_step_bytes,
            "GB/s": round(ref_step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "note": "the same step time priced with the algorithmic bytes of fprop + dgrad + wgrad as "
                    "three separate kernels (the reference's per-direction accounting)",
        },
        "fprop_frac_of_hbm_peak": kernels["fprop"]["frac_of_hbm_peak"],
        "hip_graph_replay": None if graph_ms_per_step is None else {
            "ms_per_step": round(graph_ms_per_step, 5),
            "value": round(step_bytes / (graph_ms_per_step * 1e-3) / 1e9, 1),
            "note": "the same step captured once per buffer set into a HIP graph and replayed: one graph "
                    "launch per step, whose own submission cost is not hidden behind a queue of launches "
                    "as in the eager loop",
            "steps_per_graph_many": None if long_graph_ms_per_step is None else {
                "steps_per_graph": nsets,
                "ms_per_step": round(long_graph_ms_per_step, 5),
                "value": round(step_bytes / (long_graph_ms_per_step * 1e-3) / 1e9, 1),
            },
        },
        "kernels": kernels,
        "roofline": roofline,
    }
    if not args.no_torch_gpu_baseline:
        result["torch_gpu_conv2d"] = torch_gpu_conv2d(params, sets, w, min(iters, 50))
    del sets
    torch.cuda.empty_cache()
    result["copy_ceiling"] = copy_ceiling(act_bytes, device, iters)
    best = result["copy_ceiling"]["best"]["GB/s"]
    result["roofline"]["frac_of_copy_ceiling"] = round(kernels[dominant]["GB/s"] / best, 4)
    two_one = result["copy_ceiling"]["two_in_one_out"]["best"]
    if two_one and "bgrad" in kernels:
        result["bgrad_frac_of_two_in_one_out_stream"] = round(kernels["bgrad"]["GB/s"] / two_one["GB/s"], 4)
    result["fprop_frac_of_copy_ceiling"] = round(kernels["fprop"]["GB/s"] / best, 4)
    if not args.no_cpu_baseline:
        torch.cuda.empty_cache()
        result["cpu_baseline"] = cpu_baseline(pkw, seed, args.cpu_sample_batch)
    return result


class _Skip(Exception):
    """Raised to leave out an optional measurement."""


def bench_batch_sweep(args, device, full=True):
    """cfg4: the forward kernel (and the backward half) at C=64 56x56 3x3 for N = 1 .. 512: the
    reference's headline plot, effective bandwidth versus batch size
    (scripts/profile_blocks.bash:4-5, scripts/plot_kernel_bench.py:417-435)."""
    import torch

    from spio_amd.functional import fused_backward_kernel
    from spio_amd.kernels import (
        Conv2dGw8Params,
        Conv2dStats,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )

    sweep = []
    for n in SWEEP_BATCHES:
        params = Conv2dGw8Params(n=n, c=64, h=56, w=56, padding=1, r=3, s=3)
        act = 2 * n * 64 * 56 * 56
        nsets = rotation_sets(2 * act)
        w, sets = make_buffers(params, 0, nsets, device)
        iters = 200
        min_seconds = MIN_TIMED_SECONDS if full else MIN_TIMED_SECONDS / 4
        k_fwd = conv2d_gw8_kernel_factory.get_kernel(params, device)
        fb = Conv2dStats(params, output_names="output").bytes
        e = kernel_entry(k_fwd, [(s["y"], s["x"], w, None) for s in sets], fb, iters, min_seconds)
        point = {"N": n, "fprop_us": e["us"], "fprop_GB/s": e["GB/s"], "fprop_frac": e["frac_of_hbm_peak"],
                 "fprop_bytes": fb, "launch_floor_dominated": e["us"] < 3 * LAUNCH_FLOOR_US,
                 "fprop_launch_floor_share": round(LAUNCH_FLOOR_US / e["us"], 3),
                 "fprop_frac_of_stream_model": stream_model(e["us"], fb)["frac_of_stream_model"]}  # fmt: skip
        k_fused = fused_backward_kernel(params, device)
        st_w = Conv2dStats(params, output_names="grad_weight")
        wb = st_w.bytes_read + st_w.grad_weight_bytes_written_fp32
        db = Conv2dStats(params, output_names="grad_input").bytes
        if k_fused is not None:
            bb = db + wb - act
            b = kernel_entry(k_fused, [(s["dx"], s["dw"], s["x"], s["dy"], w) for s in sets], bb, iters, min_seconds)
            point.update({"backward": "fused", "backward_us": b["us"], "backward_GB/s": b["GB/s"],
                          "backward_frac": b["frac_of_hbm_peak"], "backward_bytes": bb})  # fmt: skip
        else:
            k_d = conv2d_gw8_kernel_factory.get_kernel(params, device, igrad=True)
            k_w = conv2d_gw8_wgrad_kernel_factory.get_kernel(params, device)
            d = kernel_entry(k_d, [(s["dx"], s["dy"], w, None) for s in sets], db, iters, min_seconds)
            ww = kernel_entry(k_w, [(s["dw"], s["x"], s["dy"]) for s in sets], wb, iters, min_seconds)
            us = d["us"] + ww["us"]
            point.update({"backward": "dgrad+wgrad", "backward_us": round(us, 2),
                          "backward_GB/s": round((db + wb) / us / 1e3, 1),
                          "backward_frac": round((db + wb) / us / 1e3 / HBM_PEAK_GBS, 4),
                          "backward_bytes": db + wb})  # fmt: skip
        sweep.append(point)
        del sets
        torch.cuda.empty_cache()
    at128 = next(p for p in sweep if p["N"] == 128)
    best = max(sweep, key=lambda p: p["fprop_GB/s"])
    return {
        "metric": METRIC,
        "value": at128["fprop_GB/s"],
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(at128["fprop_us"] * 1e-3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "cfg4: conv2d_gw8 forward (and backward) C=64 56x56 3x3 pad1 fp16 NHWC, "
                               "N in {1..512}; value is the forward kernel at N=128"},
        "frac_of_hbm_peak": at128["fprop_frac"],
        "sweep": sweep,
        "roofline": {"bound": "hbm", "kernel": f"spio_conv2d_gw8_fprop at N={best['N']}",
                     "achieved": best["fprop_GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": best["fprop_frac"], "traffic": None},
        "note": f"launch_floor_dominated marks points under {3 * LAUNCH_FLOOR_US:.1f} us: an empty kernel "
                f"takes {LAUNCH_FLOOR_US} us in the same back-to-back loop",
    }  # fmt: skip


def bench_network(args, device, full=True):
    """cfg5: inference of the ConvNeXt-Tiny-shaped gw8 network at batch 128 (fp16 autocast, channels_last),
    with the time of its four distinct gw8 convolution shapes and of the channel LayerNorm."""
    import torch

    from spio_amd.convnext_gw8 import ConvNeXtGw8

    from spio_amd.kernels import Conv2dGw8Params, Conv2dStats, conv2d_gw8_kernel_factory
    from spio_amd.layers import Conv2dGw8, LayerNorm2d
    from spio_amd.kernels.layernorm_2d_kernel import (
        LayerNorm2dParams,
        layernorm_2d_bwd_kernel_factory,
        layernorm_2d_kernel_factory,
    )

    batch = 128
    torch.manual_seed(3)
    # eps = 1e-6 as in ConvNeXt: the LayerNorm shapes the packaged tuning records cover
    model = ConvNeXtGw8(make_conv=lambda dim: Conv2dGw8(dim, dim, 3, padding=1, groups=dim // 8),
                        norm2d=lambda dim: LayerNorm2d(dim, eps=1e-6))  # fmt: skip
    model = model.to(device).to(memory_format=torch.channels_last).eval()  # fp32 parameters, fp16 autocast
    gen = torch.Generator().manual_seed(3)
    images = [torch.randn(batch, 3, 224, 224, generator=gen).half().to(device)
              .contiguous(memory_format=torch.channels_last) for _ in range(2)]  # fmt: skip
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.float16):
        t0 = time.perf_counter()
        model(images[0])
        torch.cuda.synchronize()
        first_s = time.perf_counter() - t0
        for i in range(3):
            model(images[i % 2])
        torch.cuda.synchronize()
        iters = max(5, min(args.steps, 20))

        def block():
            t = time.perf_counter()
            for i in range(iters):
                model(images[i % 2])
            torch.cuda.synchronize()
            return time.perf_counter() - t

        blocks = timed_blocks(block, min_seconds=1.0 if full else 0.3, max_blocks=20)
    ms_iter = statistics.median(blocks) * 1e3 / iters

    convs, total_bytes, total_us = [], 0, 0.0
    depth = {96: 3, 192: 3, 384: 9, 768: 3}
    for c, hw in NETWORK_WIDTHS:
        params = Conv2dGw8Params(n=batch, c=c, h=hw, w=hw, padding=1, r=3, s=3, has_bias=True)
        nb = Conv2dStats(params, output_names="output").bytes
        nsets = rotation_sets(nb)
        k = conv2d_gw8_kernel_factory.get_kernel(params, device)
        asets = [conv2d_gw8_kernel_factory.make_test_args(params, device) for _ in range(nsets)]
        e = kernel_entry(k, asets, nb, 100, MIN_TIMED_SECONDS if full else MIN_TIMED_SECONDS / 4)
        e["launch_floor_share"] = round(LAUNCH_FLOOR_US / e["us"], 3)
        convs.append({"shape": params.encode(), "count": depth[c], "us": e["us"], "GB/s": e["GB/s"],
                      "frac_of_hbm_peak": e["frac_of_hbm_peak"], "bytes": nb,
                      "launch_floor_share": e["launch_floor_share"], **stream_model(e["us"], nb)})  # fmt: skip
        total_bytes += depth[c] * nb
        total_us += depth[c] * e["us"]
        del asets
        torch.cuda.empty_cache()
    norms = []
    for c, hw in NETWORK_WIDTHS:
        p = LayerNorm2dParams(n=batch, c=c, h=hw, w=hw)
        k = layernorm_2d_kernel_factory.get_kernel(p, device)
        nb = 4 * batch * c * hw * hw + 8 * c
        nsets = rotation_sets(nb)
        asets = [layernorm_2d_kernel_factory.make_test_args(p, device) for _ in range(nsets)]
        e = kernel_entry(k, asets, nb, 100, MIN_TIMED_SECONDS if full else MIN_TIMED_SECONDS / 4)
        entry = {"shape": p.encode(), "us": e["us"], "GB/s": e["GB/s"],
                 "frac_of_hbm_peak": e["frac_of_hbm_peak"], "bytes": nb}  # fmt: skip
        del asets
        torch.cuda.empty_cache()
        # its backward kernel (grad_input + partial sums of grad_weight / grad_bias): 4 B in, 2 B out
        pb = LayerNorm2dParams(n=batch, c=c, h=hw, w=hw, has_bias=False)
        kb = layernorm_2d_bwd_kernel_factory.get_kernel(pb, device)
        nbb = 6 * batch * c * hw * hw + 4 * c
        nsets = rotation_sets(nbb)
        asets = [layernorm_2d_bwd_kernel_factory.make_test_args(pb, device) for _ in range(nsets)]
        eb = kernel_entry(kb, asets, nbb, 100, MIN_TIMED_SECONDS if full else MIN_TIMED_SECONDS / 4)
        entry["backward"] = {"us": eb["us"], "GB/s": eb["GB/s"], "frac_of_hbm_peak": eb["frac_of_hbm_peak"],
                             "bytes": nbb}  # fmt: skip
        norms.append(entry)
        del asets
        torch.cuda.empty_cache()
    value = total_bytes / (total_us * 1e-6) / 1e9
    slowest = min(convs, key=lambda cv: cv["frac_of_hbm_peak"])
    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_iter, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "cfg5: ConvNeXt-Tiny-shaped network, 3x3 gw8 convolutions, batch 128, 224x224 "
                               "inference; value is the 18 gw8 convolutions' bytes over their kernel time",
                   "first_use_seconds": round(first_s, 2)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "network_ms_per_iter": round(ms_iter, 3),
        "images_per_second": round(batch / (ms_iter * 1e-3), 1),
        "gw8_conv_ms_per_iter": round(total_us * 1e-3, 3),
        "convs": convs,
        "layernorm_2d": norms,
        "roofline": {"bound": "hbm", "kernel": "spio_conv2d_gw8_fprop__" + slowest["shape"],
                     "achieved": slowest["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": slowest["frac_of_hbm_peak"], "traffic": None},
    }  # fmt: skip
    if full and not args.no_cpu_baseline:
        sample = 2
        torch.manual_seed(3)
        cpu_model = ConvNeXtGw8().float().eval()
        xs = torch.randn(sample, 3, 224, 224, generator=torch.Generator().manual_seed(3))
        with torch.no_grad():
            cpu_model(xs)
            times = []
            t_end = time.perf_counter() + 15.0
            while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 20):
                t0 = time.perf_counter()
                cpu_model(xs)
                times.append(time.perf_counter() - t0)
        med = statistics.median(times)
        result["cpu_baseline"] = {
            "value": round(sample / med, 2), "unit": "images/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"the same network with nn.Conv2d(groups=C/8) in fp32 on the host, batch {sample} of "
                      f"{batch}, median of {len(times)} passes, {med * 1e3:.0f} ms/pass",
            "logical_cpus": os.cpu_count(), "physical_cores": physical_cores(),
        }  # fmt: skip
    return result


def precompile_recorded_kernels():
    """Compiles, in the compiler's thread pool, the recorded configuration of every kernel the
    `configs` block will ask for; the code objects land in the on-disk cache, so the requests
    that follow load them instead of compiling one after the other."""
    from spio_amd.compiler.compiler_pool import compile_kernels
    from spio_amd.hip import get_device_attributes
    from spio_amd.kernels import (
        Conv2dGw8Params,
        conv2d_gw8_bgrad_kernel_factory,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )
    from spio_amd.kernels.layernorm_2d_kernel import (
        LayerNorm2dParams,
        layernorm_2d_bwd_kernel_factory,
        layernorm_2d_kernel_factory,
    )
    from spio_amd.kernels.tuner import tuner

    attr = get_device_attributes(0)
    conv_families = ((conv2d_gw8_kernel_factory, {}), (conv2d_gw8_kernel_factory, {"igrad": True}),
                     (conv2d_gw8_wgrad_kernel_factory, {}), (conv2d_gw8_bgrad_kernel_factory, {}))  # fmt: skip
    requests = []
    shapes = [Conv2dGw8Params(**WORKLOADS[w][1]) for w in ("cfg1", "cfg2", "cfg3")]
    shapes += [Conv2dGw8Params(n=n, c=64, h=56, w=56, padding=1, r=3, s=3) for n in SWEEP_BATCHES]
    for params in shapes:
        requests += [(f, params, kw) for f, kw in conv_families]
    for c, hw in NETWORK_WIDTHS:
        requests.append((conv2d_gw8_kernel_factory, Conv2dGw8Params(n=128, c=c, h=hw, w=hw, padding=1, has_bias=True), {}))
        requests.append((layernorm_2d_kernel_factory, LayerNorm2dParams(n=128, c=c, h=hw, w=hw), {}))
        requests.append((layernorm_2d_bwd_kernel_factory, LayerNorm2dParams(n=128, c=c, h=hw, w=hw, has_bias=False), {}))
    kernels = []
    for factory, params, kw in requests:
        try:
            record = tuner.lookup(attr, factory.get_full_kernel_name(params, **kw))
            if record is None:
                continue
            config = factory.config_cls(**record["config"])
            if config in list(factory.configs(params, attr, **kw)):
                kernels.append(factory.make_kernel(params, config, attr, **kw))
        except Exception:  # pylint: disable=broad-except
            continue
    try:
        compile_kernels(kernels)
    except ValueError as e:
        print(f"bench.py: precompilation failed, kernels compile on first use: {e}", file=sys.stderr)
    return len(kernels)


def configs_block(args, device):
    """Compact measurements of every benchmark configuration (cfg1..cfg5) next to the headline workload."""
    import torch

    t0 = time.perf_counter()
    out = {"precompiled_kernels": precompile_recorded_kernels()}
    out["precompile_seconds"] = round(time.perf_counter() - t0, 1)
    for name in ("cfg1", "cfg2", "cfg3"):
        t = time.perf_counter()
        try:
            out[name] = bench_conv(args, device, workload=name, full=False)
            out[name]["seconds"] = round(time.perf_counter() - t, 1)
        except Exception as e:  # pylint: disable=broad-except
            out[name] = {"error": f"{type(e).__name__}: {e}"[:300]}
        torch.cuda.empty_cache()
    t = time.perf_counter()
    try:
        sweep = bench_batch_sweep(args, device, full=False)
        out["cfg4"] = {"workload": sweep["config"]["workload"], "sweep": sweep["sweep"], "note": sweep["note"],
                       "seconds": round(time.perf_counter() - t, 1)}  # fmt: skip
    except Exception as e:  # pylint: disable=broad-except
        out["cfg4"] = {"error": f"{type(e).__name__}: {e}"[:300]}
    torch.cuda.empty_cache()
    t = time.perf_counter()
    try:
        net = bench_network(args, device, full=False)
        out["cfg5"] = {k: net[k] for k in ("network_ms_per_iter", "images_per_second", "gw8_conv_ms_per_iter",
                                           "convs", "layernorm_2d", "frac_of_hbm_peak")}  # fmt: skip
        out["cfg5"]["workload"] = net["config"]["workload"]
        out["cfg5"]["seconds"] = round(time.perf_counter() - t, 1)
    except Exception as e:  # pylint: disable=broad-except
        out["cfg5"] = {"error": f"{type(e).__name__}: {e}"[:300]}
    torch.cuda.empty_cache()
    out["seconds"] = round(time.perf_counter() - t0, 1)
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(
            "bench.py measures one GPU: the conv2d_gw8 path has no multi-GPU component "
            f"(--gpus {args.gpus} is not supported; run with --gpus 1).",
            file=sys.stderr,
        )
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False).", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    if args.workload == "cfg4":
        result = bench_batch_sweep(args, device)
    elif args.workload == "cfg5":
        result = bench_network(args, device)
    else:
        result = bench_conv(args, device)
        if args.workload == "target" and not args.no_configs:
            result["configs"] = configs_block(args, device)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
