#!/usr/bin/env python3
"""Benchmark of the conv2d_gw8 hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: the
forward kernel, the data-gradient kernel and the weight-gradient kernel
(including the zero fill of grad_weight it accumulates into) of one
convolution shape, launched through the C ABI on torch's current stream with
every tensor already resident in HBM.  Launches rotate over several buffer
sets that together exceed the 256 MB memory-side cache, so the rates are HBM
rates, not cache hits.

The single JSON line printed at the end reports
  value      effective GB/s of the whole step = algorithmic bytes of the three
             directions / step time (higher is better); the backward half runs as the
             product's backward op runs it (fused dgrad+wgrad kernel where that is faster),
  kernels    per-kernel us, effective GB/s and fraction of the 8 TB/s roofline,
             timed with HIP events on the launch stream,
  roofline   the same for the kernel that takes the most time,
  copy_yardstick  a plain non-temporal copy of the same volume (what HBM gives a read-X/write-X
             kernel on this device),
  torch_gpu_conv2d  torch's own grouped conv2d (MIOpen) on the same GPU and shapes,
  cpu_baseline  the reference's CPU oracle path (torch conv2d fp32, groups=C/8,
             and its autograd) on the host cores for a bounded sample.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload target|cfg1|cfg2|cfg3]
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what
# the same counter reads for the plain copy kernel (profiles/conv2d_gw8_target_hbm_traffic.md).
MEASURED_TRAFFIC_BYTES = {
    ("target", "fprop"): 104_710_000,
    ("target", "dgrad"): 104_720_000,
    ("target", "wgrad"): 105_510_000,
    ("target", "bgrad"): 163_270_000,
}
CACHE_BYTES = 256 * 1024 * 1024

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


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="target", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-torch-gpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-batch", type=int, default=8)
    return ap.parse_args()


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


def copy_yardstick(nbytes, nsets, device, iters):
    """Rate of a plain 16-byte-per-lane non-temporal copy of `nbytes` in and `nbytes` out."""
    import torch

    from spio_amd.compiler.compile_kernel import compile_and_load_kernel

    _module, fn = compile_and_load_kernel("spio_stream_copy", "stream_copy.hip", {}, device.index or 0)
    n = nbytes // 16
    sets = []
    for _ in range(nsets):
        src = torch.randint(0, 2**31 - 1, (n * 4,), dtype=torch.int32, device=device)
        sets.append((torch.empty_like(src), src, n))
    stream = torch.cuda.current_stream(device).cuda_stream
    ms = fn.launch_timed(((n + 255) // 256, 1, 1), (256, 1, 1), sets, 0, stream, 5, iters)
    del sets
    return {
        "kernel": "spio_stream_copy",
        "us": round(ms * 1e3, 2),
        "bytes": 2 * n * 16,
        "GB/s": round(2 * n * 16 / (ms * 1e-3) / 1e9, 1),
        "note": "plain non-temporal copy of one activation tensor in and one out: the HBM rate "
                "a read-X/write-X kernel reaches on this device",
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


def cpu_baseline(params_kwargs, seed, sample_batch):
    """The reference's oracle path on the host cores, on a bounded sample of the workload."""
    import torch

    from oracle import conv2d_gw8_oracle as oracle
    from spio_amd.kernels import Conv2dGw8Params, Conv2dStats

    kw = dict(params_kwargs)
    kw["n"] = min(kw["n"], sample_batch)
    p = Conv2dGw8Params(**kw)
    x, w, _b, dy = oracle.make_args(p.n, p.c, p.h, p.w, p.r, p.s, p.padding_h, p.padding_w, False, seed)
    threads = torch.get_num_threads()

    def one_pass():
        oracle.fprop_torch(x, w, None, p.padding_h, p.padding_w)
        oracle.grads_torch(x, w, None, dy, p.padding_h, p.padding_w)

    one_pass()
    times = []
    t_end = time.perf_counter() + 15.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 30):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    stats = Conv2dStats(p, output_names=["output", "grad_input", "grad_weight"])
    return {
        "value": round(stats.bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": (
            f"torch.nn.functional.conv2d fp32 groups=C/8 forward + autograd grads (the function the "
            f"reference's tests use as oracle), batch {p.n} of {params_kwargs['n']} of the same "
            f"workload, median of {len(times)} passes, {med * 1e3:.1f} ms/pass, "
            f"{os.cpu_count()} logical CPUs visible"
        ),
        "ms_per_pass": round(med * 1e3, 3),
    }


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

    from spio_amd.kernels import (
        Conv2dGw8Params,
        Conv2dStats,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )

    desc, pkw, seed = WORKLOADS[args.workload]
    params = Conv2dGw8Params(**pkw)
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    set_bytes = 2 * (2 * params.n * params.c * params.h * params.w + 2 * params.n * params.c * params.p * params.q)
    nsets = max(2, min(8, -(-3 * CACHE_BYTES // set_bytes)))
    w, sets = make_buffers(params, seed, nsets, device)

    # First use: tunes (or reads the recorded choice), compiles and loads.
    t0 = time.perf_counter()
    k_fwd = conv2d_gw8_kernel_factory.get_kernel(params, device)
    k_dgrad = conv2d_gw8_kernel_factory.get_kernel(params, device, igrad=True)
    k_wgrad = conv2d_gw8_wgrad_kernel_factory.get_kernel(params, device)
    setup_s = time.perf_counter() - t0

    # The backward half of the step runs the way the product's backward op runs it: one fused
    # data+weight gradient kernel where the recorded times say it beats the two separate ones.
    from spio_amd.functional import fused_backward_kernel

    k_fused = fused_backward_kernel(params, device)

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
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # The same steps replayed from HIP graphs (one graph per buffer set): what a caller that
    # captures its training step gets; reported beside the eager figure, which stays `value`.
    graph_ms_per_step = None
    try:
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
        t0 = time.perf_counter()
        for i in range(args.steps):
            graphs[i % nsets].replay()
        torch.cuda.synchronize()
        graph_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        del graphs
    except Exception as e:  # pylint: disable=broad-except
        print(f"bench.py: HIP graph replay skipped: {type(e).__name__}: {e}", file=sys.stderr)

    # Per-kernel times with HIP events on the launch stream.
    iters = max(20, min(args.steps, 200))
    st = {
        "fprop": Conv2dStats(params, output_names="output"),
        "dgrad": Conv2dStats(params, output_names="grad_input"),
        "wgrad": Conv2dStats(params, output_names="grad_weight"),
    }
    arg_sets = {
        "fprop": (k_fwd, [(s["y"], s["x"], w, None) for s in sets]),
        "dgrad": (k_dgrad, [(s["dx"], s["dy"], w, None) for s in sets]),
        "wgrad": (k_wgrad, [(s["dw"], s["x"], s["dy"]) for s in sets]),
    }
    kernels = {}
    for name, (kernel, asets) in arg_sets.items():
        ms = kernel.time(asets, warmup=5, iters=iters)
        nbytes = st[name].bytes
        if name == "wgrad":  # grad_weight is fp32 on the device
            nbytes = st[name].bytes_read + st[name].grad_weight_bytes_written_fp32
        gbs = nbytes / (ms * 1e-3) / 1e9
        kernels[name] = {
            "us": round(ms * 1e3, 2),
            "bytes": nbytes,
            "GB/s": round(gbs, 1),
            "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "config": {k: v for k, v in vars(kernel.config).items()},
            "kernel": kernel.kernel_name,
        }
    # `value` keeps the reference's accounting (the algorithmic bytes of the three directions,
    # scripts/plot_kernel_bench.py:430-435) whether or not the backward half is fused, so it is a
    # pure time metric; the fused kernel's own roofline entry counts grad_output once.
    step_bytes = sum(k["bytes"] for k in kernels.values())
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    if k_fused is not None:
        ms = k_fused.time([(s["dx"], s["dw"], s["x"], s["dy"], w) for s in sets], warmup=5, iters=iters)
        nbytes = (st["dgrad"].bytes + st["wgrad"].bytes_read + st["wgrad"].grad_weight_bytes_written_fp32
                  - 2 * params.n * params.c * params.p * params.q)  # grad_output is read once
        gbs = nbytes / (ms * 1e-3) / 1e9
        kernels["bgrad"] = {
            "us": round(ms * 1e3, 2),
            "bytes": nbytes,
            "GB/s": round(gbs, 1),
            "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "config": {k: v for k, v in vars(k_fused.config).items()},
            "kernel": k_fused.kernel_name,
            "note": "fused dgrad+wgrad as the backward op runs it for this shape; replaces the "
                    "dgrad and wgrad launches in the timed step",
            # the same time priced with the bytes the two separate kernels need for this work
            "unfused_accounting": {
                "bytes": kernels["dgrad"]["bytes"] + kernels["wgrad"]["bytes"],
                "GB/s": round((kernels["dgrad"]["bytes"] + kernels["wgrad"]["bytes"]) / (ms * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(
                    (kernels["dgrad"]["bytes"] + kernels["wgrad"]["bytes"]) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4
                ),
            },
        }

    in_step = [n for n in kernels if (n in ("fprop", "bgrad") if k_fused is not None else n != "bgrad")]
    dominant = max(in_step, key=lambda n: kernels[n]["us"])
    roofline = {
        "bound": "hbm",
        "kernel": kernels[dominant]["kernel"],
        "achieved": kernels[dominant]["GB/s"],
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": kernels[dominant]["frac_of_hbm_peak"],
        "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, dominant)),
    }

    result = {
        "metric": "conv2d_gw8 effective HBM bandwidth (fwd+dgrad+wgrad step)",
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
        },
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "value_note": "algorithmic bytes of fprop + dgrad + wgrad (the reference's per-direction accounting) "
                      "divided by the time of one step as the operators run it"
                      + ("; the backward half of this step is one fused kernel that reads grad_output once, "
                         "so the step moves fewer bytes than the numerator counts" if k_fused is not None else ""),
        "hip_graph_replay": None if graph_ms_per_step is None else {
            "ms_per_step": round(graph_ms_per_step, 5),
            "value": round(step_bytes / (graph_ms_per_step * 1e-3) / 1e9, 1),
            "note": "the same step captured once per buffer set into a HIP graph and replayed",
        },
        "kernels": kernels,
        "roofline": roofline,
    }
    if not args.no_torch_gpu_baseline:
        result["torch_gpu_conv2d"] = torch_gpu_conv2d(params, sets, w, min(iters, 50))
    del arg_sets
    del sets
    torch.cuda.empty_cache()
    result["copy_yardstick"] = copy_yardstick(
        2 * params.n * params.c * params.h * params.w, nsets, device, iters
    )
    result["roofline"]["frac_of_copy_rate"] = round(
        kernels[dominant]["GB/s"] / result["copy_yardstick"]["GB/s"], 4
    )
    if not args.no_cpu_baseline:
        torch.cuda.empty_cache()
        result["cpu_baseline"] = cpu_baseline(pkw, seed, args.cpu_sample_batch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
