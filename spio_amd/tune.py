"""Command-line tuning: run the on-device sweep for a list of shapes and record the choices.

    python -m spio_amd.tune --shapes bench            # the benchmark shapes
    python -m spio_amd.tune 128n_64c_56h_56w_1py_1px_3r_3s_nb [...]
    python -m spio_amd.tune 128n_96c_56h_56w_1em06eps_wb      # a LayerNorm2d shape
    python -m spio_amd.tune --shapes bench --package  # write into the package's own records

Records land in the user cache (or SPIO_TUNE_DB) unless --package is given; later processes
read them and compile only the chosen configuration.  This takes the place of the reference's
performance-model training scripts (scripts/train_performance_model.py): the choice is measured
per shape instead of predicted.
"""

import argparse
import os
import sys
from typing import Any, Dict, List, Optional, Sequence

BENCH_SHAPES = [
    "32n_64c_56h_56w_1py_1px_3r_3s_nb",
    "128n_64c_56h_56w_1py_1px_3r_3s_nb",
    "128n_128c_28h_28w_1py_1px_3r_3s_nb",
    "256n_256c_14h_14w_3py_3px_7r_7s_nb",
]
# rows wider than the LDS rings hold whole: the kernels tile them into column blocks
WIDE_SHAPES = [
    "16n_64c_128h_512w_1py_1px_3r_3s_nb",
    "8n_64c_64h_1024w_1py_1px_3r_3s_nb",
    "32n_64c_224h_224w_1py_1px_3r_3s_nb",
]
SWEEP_BATCHES = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]
NETWORK_SHAPES = [
    "128n_96c_56h_56w_1py_1px_3r_3s_b",
    "128n_192c_28h_28w_1py_1px_3r_3s_b",
    "128n_384c_14h_14w_1py_1px_3r_3s_b",
    "128n_768c_7h_7w_1py_1px_3r_3s_b",
    # the channel LayerNorms of the same network (LayerNorm2dParams.encode() form)
    "128n_96c_56h_56w_1em06eps_wb",
    "128n_192c_28h_28w_1em06eps_wb",
    "128n_384c_14h_14w_1em06eps_wb",
    "128n_768c_7h_7w_1em06eps_wb",
]


def tune_model(model, inputs: Sequence, backward: bool = True, max_configs: Optional[int] = 8,
               iters: int = 5, warmup: int = 2, record_path: Optional[str] = None, record: bool = True,
               autocast_dtype=None, loss=None) -> List[Dict[str, Any]]:  # fmt: skip
    """Tune the kernels a model actually asks for, inside the model.

    Takes the place of the reference's benchmarking harness (scripts/profile_block.py:545-701):
      1. one forward (+ backward) pass under `KernelParamsLogger` records every
         (kernel factory, params, kwargs) the model requests;
      2. the candidate configurations of exactly those kernels are compiled (the `max_configs`
         best-ranked ones of each; None = all);
      3. round i pins the i-th candidate of every kernel through the caches' overlays
         (`KernelCache.update_overlay`) and runs the model `warmup + iters` times over `inputs`
         (a list of input batches, rotated) while `LaunchTimer` times each launch with HIP events:
         kernels are timed with the cache state and neighbours they have in the model;
      4. every round's model output and, with `backward`, the gradients of the model's
         parameters after its first iteration are kept; the rounds are then compared with each
         other and those that disagree with the largest group of agreeing rounds are discarded
         as a whole (one of their configurations computes something else, in the forward or in
         the backward pass; a wrong first round is outvoted like any other);
      5. the fastest candidate of every kernel is written to the tuning records (the user
         record file, or `record_path`), the caches are cleared, and the next request for each
         of these kernels compiles the recorded winner.

    Returns one dict per kernel: name, chosen config, its microseconds, and all timed candidates.
    """
    import torch

    from .compiler.compiler_pool import compile_kernel_configs
    from .functional import reset_fused_backward_choices
    from .hip import get_device_attributes
    from .kernels.kernel import LaunchTimer
    from .kernels.kernel_params_logger import KernelParamsLogger
    from .kernels.tuner import config_to_dict, tuner

    inputs = list(inputs) if isinstance(inputs, (list, tuple)) else [inputs]
    if loss is None:
        loss = lambda out: out.float().sum()  # noqa: E731

    def run(x):
        ctx = torch.autocast(device_type="cuda", dtype=autocast_dtype) if autocast_dtype else _NullContext()
        if backward:
            with ctx:
                out = model(x)
            loss(out).backward()
            return out.detach()
        with torch.no_grad(), ctx:
            return model(x)

    # 1. what does the model ask for?  (remembered fused/separate choices would hide requests)
    reset_fused_backward_choices()
    with KernelParamsLogger() as logger:
        run(inputs[0])
        torch.cuda.synchronize()
    unique = list(dict.fromkeys(logger.get_logged_params()))
    if not unique:
        return []
    caches = {id(kp.kernel_cache): kp.kernel_cache for kp in unique}
    for cache in caches.values():
        cache.clear_cache()
    reset_fused_backward_choices()

    # 2. candidates
    table = {}
    for kp in unique:
        attr = get_device_attributes(kp.key.device_ordinal)
        kwargs = dict(kp.kernel_kwargs)
        configs = list(kp.kernel_factory.configs(kp.params, attr, **kwargs))
        if max_configs is not None:
            configs = configs[:max_configs]
        table[kp] = compile_kernel_configs(kp.kernel_factory, kp.params, configs=configs, device_attr=attr, **kwargs)
    rounds = max(len(kernels) for kernels in table.values())

    # 3./4. rounds with pinned configurations.  Where the model's backward pass can run either the
    # fused data+weight gradient kernel or the two separate ones, every round is run both ways so
    # that all three families get their in-situ times.
    times: Dict[Any, Dict[int, float]] = {kp: {} for kp in unique}
    round_times = []  # (idx, mode, {kp: us}) per round
    round_results = []  # what the model computed in that round: [output, gradients...]
    discarded = []
    has_fused = any(kp.kernel_factory.get_kernel_name(**dict(kp.kernel_kwargs)).endswith("bgrad") for kp in unique)
    saved_mode = os.environ.get("SPIO_FUSED_BACKWARD")
    passes = [(idx, mode) for idx in range(rounds) for mode in (("1", "0") if has_fused and backward else (None,))]
    for idx, mode in passes:
        if mode is not None:
            os.environ["SPIO_FUSED_BACKWARD"] = mode
        choice = {kp: kernels[idx % len(kernels)] for kp, kernels in table.items()}
        overlays: Dict[int, Dict[Any, Any]] = {}
        for kp, kernel in choice.items():
            overlays.setdefault(id(kp.kernel_cache), {})[kp.key] = kernel
            kernel.load(kp.key.device_ordinal, clear_code=False)
        for cid, overlay in overlays.items():
            caches[cid].update_overlay(overlay)
        reset_fused_backward_choices()
        try:
            if backward:
                model.zero_grad(set_to_none=True)
            with LaunchTimer() as timer:
                for i in range(warmup + iters):
                    out = run(inputs[i % len(inputs)])
                    if i == 0:
                        computed = [out.float().clone()]
                        if backward:
                            computed += [p.grad.float().clone() for p in model.parameters() if p.grad is not None]
                averages = timer.averages(skip=warmup)
        finally:
            for cache in caches.values():
                cache.clear_overlay()
            for kernel in choice.values():
                kernel.unload()
            if mode is not None:
                if saved_mode is None:
                    os.environ.pop("SPIO_FUSED_BACKWARD", None)
                else:
                    os.environ["SPIO_FUSED_BACKWARD"] = saved_mode
        round_results.append(computed)
        round_times.append((idx, mode, {kp: averages[kernel] for kp, kernel in choice.items()
                                        if idx < len(table[kp]) and kernel in averages}))  # fmt: skip

    def agree(a, b):
        return len(a) == len(b) and all(
            x.shape == y.shape and torch.allclose(x, y, rtol=2e-2, atol=2e-2 * max(float(y.abs().max()), 1e-6))
            for x, y in zip(a, b)
        )

    # the reference is the round most other rounds agree with
    votes = [sum(agree(a, b) for b in round_results) for a in round_results]
    reference = round_results[votes.index(max(votes))]
    for (idx, mode, per_kernel), computed in zip(round_times, round_results):
        if not agree(computed, reference):
            discarded.append((idx, mode))
            continue
        for kp, us in per_kernel.items():
            times[kp][idx] = us
    del round_results, reference

    # 5. record the winners
    results = []
    for kp in unique:
        kernels = table[kp]
        attr = get_device_attributes(kp.key.device_ordinal)
        kwargs = dict(kp.kernel_kwargs)
        name = kp.kernel_factory.get_full_kernel_name(kp.params, **kwargs)
        timed = sorted(times[kp].items(), key=lambda it: it[1])
        entry = {"kernel": name, "candidates": len(kernels), "config": None, "us": None,
                 "sweep": [{"config": config_to_dict(kernels[i].config), "us": us} for i, us in timed]}  # fmt: skip
        if timed:
            best_idx, best_us = timed[0]
            entry["config"] = config_to_dict(kernels[best_idx].config)
            entry["us"] = best_us
            if record:
                tuner._store(attr, name, {"config": entry["config"], "us": best_us, "candidates": len(kernels),
                                          "sweep": entry["sweep"][:8], "in_situ": True}, record_path)  # fmt: skip
        results.append(entry)
        for kernel in kernels:
            kernel.code = None
    for cache in caches.values():
        cache.clear_cache()
    reset_fused_backward_choices()
    if discarded:
        print(f"spio: tune_model discarded rounds {discarded}: output or gradients differed from the other rounds")
    return results


class _NullContext:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("shapes", nargs="*", help="shapes in Conv2dGw8Params.encode() form")
    ap.add_argument("--shapes", dest="preset", choices=["bench", "batch-sweep", "network", "wide", "all"])
    ap.add_argument("--directions", default="fprop,dgrad,wgrad,bgrad",
                    help="bgrad = the fused data+weight gradient kernel")
    ap.add_argument("--iters", type=int, default=30)
    ap.add_argument("--package", action="store_true", help="write into spio_amd/kernels/tuned/")
    args = ap.parse_args(argv)

    import torch

    from .hip import get_device_attributes
    from .kernels import (
        Conv2dGw8Params,
        LayerNorm2dParams,
        conv2d_gw8_bgrad_kernel_factory,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
        layernorm_2d_bwd_is_supported,
        layernorm_2d_bwd_kernel_factory,
        layernorm_2d_kernel_factory,
    )
    from .kernels.tuner import _PACKAGE_RECORDS, device_key, tuner

    shapes = list(args.shapes)
    if args.preset in ("bench", "all"):
        shapes += BENCH_SHAPES
    if args.preset in ("batch-sweep", "all"):
        shapes += [f"{n}n_64c_56h_56w_1py_1px_3r_3s_nb" for n in SWEEP_BATCHES]
    if args.preset in ("network", "all"):
        shapes += NETWORK_SHAPES
    if args.preset in ("wide", "all"):
        shapes += WIDE_SHAPES
    if not shapes:
        ap.error("no shapes given")
    if not torch.cuda.is_available():
        sys.exit("tuning needs a GPU")
    attr = get_device_attributes(0)
    path = None
    if args.package:
        os.makedirs(_PACKAGE_RECORDS, exist_ok=True)
        path = os.path.join(_PACKAGE_RECORDS, device_key(attr) + ".json")
    families = {
        "fprop": (conv2d_gw8_kernel_factory, {}),
        "dgrad": (conv2d_gw8_kernel_factory, {"igrad": True}),
        "wgrad": (conv2d_gw8_wgrad_kernel_factory, {}),
        "bgrad": (conv2d_gw8_bgrad_kernel_factory, {}),
    }
    seen = set()
    for shape in shapes:
        if shape in seen:
            continue
        seen.add(shape)
        if "eps_" in shape:  # a LayerNorm2d shape: the forward kernel and the backward kernel
            params = LayerNorm2dParams.decode(shape)
            # the backward kernel does not depend on the bias: its records are kept without one
            bwd_params = LayerNorm2dParams(n=params.n, c=params.c, h=params.h, w=params.w, eps=params.eps,
                                           has_weight=params.has_weight, has_bias=False)  # fmt: skip
            for tag, factory, p in (("lnorm", layernorm_2d_kernel_factory, params),
                                    ("lnbwd", layernorm_2d_bwd_kernel_factory, bwd_params)):  # fmt: skip
                if tag == "lnbwd" and not layernorm_2d_bwd_is_supported(p):
                    continue
                kernel = tuner.sweep(factory, p, 0, attr, warmup=3, iters=args.iters, record_path=path)
                best = min(r["us"] for r in tuner.last_sweep if "us" in r)
                print(f"{tag} {p.encode()}: {best:8.1f} us  {kernel.config}", flush=True)
                kernel.unload()
                torch.cuda.empty_cache()
            continue
        params = Conv2dGw8Params.decode(shape)
        for direction in args.directions.split(","):
            factory, kwargs = families[direction]
            if not list(factory.configs(params, attr, **kwargs)):
                print(f"{direction:5s} {shape}: not supported", flush=True)
                continue
            kernel = tuner.sweep(factory, params, 0, attr, warmup=3, iters=args.iters,
                                 record_path=path, **kwargs)  # fmt: skip
            best = min(r["us"] for r in tuner.last_sweep if "us" in r)
            print(f"{direction:5s} {shape}: {best:8.1f} us  {kernel.config}", flush=True)
            kernel.unload()
            torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
