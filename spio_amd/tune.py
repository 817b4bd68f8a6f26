"""Command-line tuning: run the on-device sweep for a list of shapes and record the choices.

    python -m spio_amd.tune --shapes bench            # the benchmark shapes
    python -m spio_amd.tune 128n_64c_56h_56w_1py_1px_3r_3s_nb [...]
    python -m spio_amd.tune --shapes bench --package  # write into the package's own records

Records land in the user cache (or SPIO_TUNE_DB) unless --package is given; later processes
read them and compile only the chosen configuration.  This takes the place of the reference's
performance-model training scripts (scripts/train_performance_model.py): the choice is measured
per shape instead of predicted.
"""

import argparse
import os
import sys

BENCH_SHAPES = [
    "32n_64c_56h_56w_1py_1px_3r_3s_nb",
    "128n_64c_56h_56w_1py_1px_3r_3s_nb",
    "128n_128c_28h_28w_1py_1px_3r_3s_nb",
    "256n_256c_14h_14w_3py_3px_7r_7s_nb",
]
SWEEP_BATCHES = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]
NETWORK_SHAPES = [
    "128n_96c_56h_56w_1py_1px_3r_3s_b",
    "128n_192c_28h_28w_1py_1px_3r_3s_b",
    "128n_384c_14h_14w_1py_1px_3r_3s_b",
    "128n_768c_7h_7w_1py_1px_3r_3s_b",
]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("shapes", nargs="*", help="shapes in Conv2dGw8Params.encode() form")
    ap.add_argument("--shapes", dest="preset", choices=["bench", "batch-sweep", "network", "all"])
    ap.add_argument("--directions", default="fprop,dgrad,wgrad,bgrad",
                    help="bgrad = the fused data+weight gradient kernel (size-preserving shapes only)")
    ap.add_argument("--iters", type=int, default=30)
    ap.add_argument("--package", action="store_true", help="write into spio_amd/kernels/tuned/")
    args = ap.parse_args(argv)

    import torch

    from .hip import get_device_attributes
    from .kernels import (
        Conv2dGw8Params,
        conv2d_gw8_bgrad_kernel_factory,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )
    from .kernels.tuner import _PACKAGE_RECORDS, device_key, tuner

    shapes = list(args.shapes)
    if args.preset in ("bench", "all"):
        shapes += BENCH_SHAPES
    if args.preset in ("batch-sweep", "all"):
        shapes += [f"{n}n_64c_56h_56w_1py_1px_3r_3s_nb" for n in SWEEP_BATCHES]
    if args.preset in ("network", "all"):
        shapes += NETWORK_SHAPES
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
