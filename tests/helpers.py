"""Test procedures shared by the GPU parity tests.

They restate the reference's procedures (spio/src_tests/run_test.py:26-246):
run every configuration of a kernel on seeded inputs with the output
pre-filled by a sentinel, and compare with the fp32 CPU oracle.
"""

import json
import os
import random
from dataclasses import replace
from typing import List

import torch

from oracle import conv2d_gw8_oracle as oracle
from spio_amd.compiler import compile_kernel_configs
from spio_amd.hip import get_device_attributes
from spio_amd.kernels import Conv2dGw8Params, Conv2dStats

DEAD_VALUE = -42.0  # every output element must be overwritten (run_test.py:23,64)
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MAX_TEST_PARAMS = int(os.environ.get("SPIO_MAX_TEST_PARAMS", "10"))
MAX_TEST_CONFIGS = int(os.environ.get("SPIO_MAX_TEST_CONFIGS", "6"))
MAX_ORACLE_BATCH = 8


def model_shapes(has_bias=None) -> List[Conv2dGw8Params]:
    """The 81 model-derived layer shapes of the reference's corpus.

    The batch is cut to MAX_ORACLE_BATCH so the CPU oracle finishes in seconds.
    """
    with open(os.path.join(GOLDEN, "conv2d_gw8_model_shapes.json"), "r", encoding="utf-8") as f:
        rows = json.load(f)
    out = []
    for d in rows:
        out.append(
            Conv2dGw8Params(
                n=min(d["n"], MAX_ORACLE_BATCH), c=d["c"], h=d["h"], w=d["w"],
                padding=(d["py"], d["px"]), r=d["r"], s=d["s"],
                has_bias=d["has_bias"] if has_bias is None else has_bias,
            )  # fmt: skip
        )
    return out


def reference_test_params(has_bias=False) -> List[Conv2dGw8Params]:
    """The shape list of tests/test_conv2d_gw8.py:67-107 in the reference."""
    P = Conv2dGw8Params
    kw = {"has_bias": has_bias}
    rxs = [P(n=1, c=128, h=32, w=32, r=r, s=s, padding=(r // 2, s // 2), **kw)
           for r in range(1, 6) for s in range(1, 6)]  # fmt: skip
    padding = [
        P(n=1, c=128, h=64, w=64, padding=0, **kw),
        P(n=4, c=128, h=20, w=19, padding=0, **kw),
        P(n=1, c=128, h=64, w=64, padding=2, **kw),
        P(n=1, c=128, h=64, w=64, padding=7, **kw),
    ]
    groups = [P(n=4, c=g * 8, h=32, w=32, **kw) for g in range(1, 17)]
    misc = [
        P(n=6, c=128, h=49, w=33, **kw),
        P(n=6, c=128, h=6, w=5, **kw),
        P(n=8, c=1024, h=7, w=7, **kw),
        P(n=8, c=64, h=64, w=64, **kw),
        P(n=8, c=256, h=64, w=64, **kw),
        P(n=3, c=128, h=16, w=16, **kw),
        P(n=4, c=128, h=32, w=16, **kw),
        P(n=5, c=128, h=16, w=32, **kw),
        P(n=6, c=128, h=48, w=32, **kw),
    ]
    return [replace(p, **kw) for p in model_shapes()] + rxs + padding + groups + misc


def sample_params(seed: int, count: int = MAX_TEST_PARAMS) -> List[Conv2dGw8Params]:
    """Seeded random draw from the with-bias and without-bias shape lists."""
    pool = reference_test_params(True) + reference_test_params(False)
    if count <= 0 or count >= len(pool):
        return pool
    return random.Random(seed).sample(pool, count)


def random_params(seed: int, count: int, max_elements: int = 3_000_000) -> List[Conv2dGw8Params]:
    """Seeded random shapes beyond the reference's list: every filter size from 1x1 to 7x7 with
    r != s, padding from none to more than the filter's half, odd image sizes and batches, few
    and many groups.  Sizes stay small enough for the CPU oracle."""
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        r, s = rng.randint(1, 7), rng.randint(1, 7)
        if rng.random() < 0.3:
            r = s = rng.choice([3, 3, 5, 7])
        py = rng.choice([r // 2, r // 2, 0, rng.randint(0, r)])
        px = rng.choice([s // 2, s // 2, 0, rng.randint(0, s)])
        h = rng.choice([rng.randint(1, 20), rng.randint(1, 70), 7, 14, 28, 56])
        w = rng.choice([rng.randint(1, 20), rng.randint(1, 70), 7, 14, 28, 56, 33, 65, 96])
        n = rng.choice([1, 2, 3, 5, 8, rng.randint(1, 9)])
        c = 8 * rng.choice([1, 2, 3, 4, 5, 8, 12, 16, rng.randint(1, 24)])
        params = Conv2dGw8Params(n=n, c=c, h=h, w=w, r=r, s=s, padding=(py, px), has_bias=rng.random() < 0.5)
        if params.is_valid() and n * c * max(h * w, params.p * params.q) <= max_elements:
            out.append(params)
    return out


def pick_configs(factory, params, device_attr, configs=None, limit=MAX_TEST_CONFIGS, seed=0, **kw):
    """All given configs, or a bounded spread of the legal ones (first, last, random)."""
    if configs is not None:
        return list(configs)
    allc = list(factory.configs(params, device_attr, **kw))
    if limit <= 0 or len(allc) <= limit:
        return allc
    rng = random.Random(seed)
    keep = [allc[0], allc[1], allc[-1]]
    rest = [c for c in allc if c not in keep]
    return keep + rng.sample(rest, limit - len(keep))


def gpu_args(params: Conv2dGw8Params, seed=0, weight_init="randn"):
    x, w, bias, dy = oracle.make_args(
        params.n, params.c, params.h, params.w, params.r, params.s,
        params.padding_h, params.padding_w, params.has_bias, seed=seed, weight_init=weight_init,
    )  # fmt: skip
    return x, w, bias, dy


def to_gpu(t):
    if t is None:
        return None
    if t.dim() == 4:
        return t.cuda().contiguous(memory_format=torch.channels_last)
    return t.cuda()


def run_kernel_test(factory, params: Conv2dGw8Params, configs=None, seed=0, **kw):
    """fprop kernel: every picked configuration against the oracle."""
    attr = get_device_attributes(0)
    x, w, bias, _dy = gpu_args(params, seed)
    expected = oracle.fprop_torch(x, w, bias, params.padding_h, params.padding_w)
    depth = Conv2dStats(params, output_names="output").accumulation_depths[0]
    kernels = compile_kernel_configs(
        factory, params, configs=pick_configs(factory, params, attr, configs, **kw), device_attr=attr, **kw
    )
    xg, wg, bg = to_gpu(x), to_gpu(w), to_gpu(bias)
    for kernel in kernels:
        kernel.load(0)
        out = torch.full(params.output_shape, DEAD_VALUE, device="cuda", dtype=torch.float16).contiguous(
            memory_format=torch.channels_last
        )
        kernel(out, xg, wg, bg)
        torch.cuda.synchronize()
        oracle.check_close(out, expected, acc_depth=depth, what=f"fprop {params.encode()} {kernel.config}")
        oracle.check_close(out, expected, what=f"fprop(north-star tol) {params.encode()} {kernel.config}")
        kernel.unload()


def run_grad_kernel_test(factory, params: Conv2dGw8Params, configs=None, seed=0, igrad=False):
    """dgrad (igrad=True) or wgrad kernel: every picked configuration against the oracle."""
    attr = get_device_attributes(0)
    x, w, bias, dy = gpu_args(params, seed)
    dx_e, dw_e, _db_e = oracle.grads_torch(x, w, bias, dy, params.padding_h, params.padding_w)
    kw = {"igrad": True} if igrad else {}
    kernels = compile_kernel_configs(
        factory, params, configs=pick_configs(factory, params, attr, configs, **kw), device_attr=attr, **kw
    )
    xg, wg, dyg = to_gpu(x), to_gpu(w), to_gpu(dy)
    for kernel in kernels:
        kernel.load(0)
        if igrad:
            depth = Conv2dStats(params, output_names="grad_input").accumulation_depths[0]
            out = torch.full(params.input_shape, DEAD_VALUE, device="cuda", dtype=torch.float16).contiguous(
                memory_format=torch.channels_last
            )
            kernel(out, dyg, wg, None)
            torch.cuda.synchronize()
            oracle.check_close(out, dx_e, acc_depth=depth, what=f"dgrad {params.encode()} {kernel.config}")
        else:
            depth = Conv2dStats(params, output_names="grad_weight").accumulation_depths[0]
            out = torch.zeros(params.weight_shape, device="cuda", dtype=torch.float32).contiguous(
                memory_format=torch.channels_last
            )
            if params.has_bias:
                # with a bias the kernel also sums grad_output per channel into its fourth argument
                db = torch.zeros(params.c, device="cuda", dtype=torch.float32)
                kernel(out, xg, dyg, db)
                torch.cuda.synchronize()
                oracle.check_close(db, _db_e, acc_depth=params.n * params.p * params.q,
                                   what=f"grad_bias {params.encode()} {kernel.config}")  # fmt: skip
            else:
                kernel(out, xg, dyg)
                torch.cuda.synchronize()
            oracle.check_close(out, dw_e, acc_depth=depth, what=f"wgrad {params.encode()} {kernel.config}")
        kernel.unload()


def run_bgrad_kernel_test(factory, params: Conv2dGw8Params, configs=None, seed=0):
    """Fused backward kernel: grad_input, grad_weight (and grad_bias) of every picked
    configuration against the oracle; grad_input is pre-filled with a sentinel."""
    attr = get_device_attributes(0)
    x, w, bias, dy = gpu_args(params, seed)
    dx_e, dw_e, db_e = oracle.grads_torch(x, w, bias, dy, params.padding_h, params.padding_w)
    picked = pick_configs(factory, params, attr, configs)
    assert picked, f"no fused backward configuration for {params}"
    kernels = compile_kernel_configs(factory, params, configs=picked, device_attr=attr)
    xg, wg, dyg = to_gpu(x), to_gpu(w), to_gpu(dy)
    d_dx = Conv2dStats(params, output_names="grad_input").accumulation_depths[0]
    d_dw = Conv2dStats(params, output_names="grad_weight").accumulation_depths[0]
    for kernel in kernels:
        kernel.load(0)
        what = f"{params.encode()} {kernel.config}"
        dx = torch.full(params.input_shape, DEAD_VALUE, device="cuda", dtype=torch.float16).contiguous(
            memory_format=torch.channels_last
        )
        dw = torch.zeros(params.weight_shape, device="cuda", dtype=torch.float32).contiguous(
            memory_format=torch.channels_last
        )
        if params.has_bias:
            db = torch.zeros(params.c, device="cuda", dtype=torch.float32)
            kernel(dx, dw, xg, dyg, wg, db)
            torch.cuda.synchronize()
            oracle.check_close(db, db_e, acc_depth=params.n * params.p * params.q, what=f"fused grad_bias {what}")
        else:
            kernel(dx, dw, xg, dyg, wg)
            torch.cuda.synchronize()
        oracle.check_close(dx, dx_e, acc_depth=d_dx, what=f"fused dgrad {what}")
        oracle.check_close(dw, dw_e, acc_depth=d_dw, what=f"fused wgrad {what}")
        kernel.unload()
