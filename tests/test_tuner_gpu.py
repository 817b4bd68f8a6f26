"""The on-device configuration sweep: it runs, records its choice, and the record is reused.
GPU only."""

import json
from dataclasses import replace

import pytest
import torch

from helpers import to_gpu
from oracle import conv2d_gw8_oracle as oracle
from spio_amd.hip import get_device_attributes
from spio_amd.kernels import Conv2dGw8Params, conv2d_gw8_kernel_factory, conv2d_gw8_wgrad_kernel_factory
from spio_amd.kernels.tuner import Tuner

pytestmark = pytest.mark.gpu


def test_sweep_records_and_reuses_choice(tmp_path, monkeypatch):
    monkeypatch.setenv("SPIO_TUNE_DB", str(tmp_path / "tune.json"))
    monkeypatch.setenv("SPIO_TUNE", "1")
    attr = get_device_attributes(0)
    params = Conv2dGw8Params(n=8, c=64, h=28, w=28)
    tuner = Tuner()
    configs = list(conv2d_gw8_kernel_factory.configs(params, attr))[:6]
    kernel = tuner.sweep(conv2d_gw8_kernel_factory, params, 0, attr, configs=configs)
    assert kernel.function is not None and kernel.config in configs
    timed = [r for r in tuner.last_sweep if "us" in r]
    assert len(timed) == len(configs) and all(r["us"] > 0 for r in timed)
    name = conv2d_gw8_kernel_factory.get_full_kernel_name(params)
    record = json.load(open(tmp_path / "tune.json"))[name]
    assert record["config"] == vars(kernel.config) and record["candidates"] == len(configs)
    assert record["us"] == pytest.approx(min(r["us"] for r in timed))

    # A fresh tuner (a new process would do the same) reads the record: no sweep.
    again = Tuner()
    k2 = again.best_kernel(conv2d_gw8_kernel_factory, params, 0, attr)
    assert again.last_sweep is None and k2.config == kernel.config

    # The chosen kernel computes the right thing.
    x, w, _b, _dy = oracle.make_args(params.n, params.c, params.h, params.w, 3, 3, 1, 1, False, 0)
    y = torch.empty(params.output_shape, device="cuda", dtype=torch.float16).contiguous(memory_format=torch.channels_last)
    k2(y, to_gpu(x), to_gpu(w), None)
    torch.cuda.synchronize()
    oracle.check_close(y, oracle.fprop_torch(x, w, None, 1, 1), acc_depth=72, what="tuned kernel")


def test_wgrad_sweep_covers_both_publish_modes(tmp_path, monkeypatch):
    monkeypatch.setenv("SPIO_TUNE_DB", str(tmp_path / "tune.json"))
    attr = get_device_attributes(0)
    params = Conv2dGw8Params(n=8, c=64, h=28, w=28)
    configs = list(conv2d_gw8_wgrad_kernel_factory.configs(params, attr))
    first = next(c for c in configs if c.variant == "mfma")
    one = replace(first, two_stage=0)
    two = replace(first, two_stage=1)
    tuner = Tuner()
    kernel = tuner.sweep(conv2d_gw8_wgrad_kernel_factory, params, 0, attr, configs=[one, two, configs[-1]])
    assert len([r for r in tuner.last_sweep if "us" in r]) == 3
    x, w, _b, dy = oracle.make_args(params.n, params.c, params.h, params.w, 3, 3, 1, 1, False, 1)
    dw = torch.zeros(params.weight_shape, device="cuda").contiguous(memory_format=torch.channels_last)
    kernel(dw, to_gpu(x), to_gpu(dy))
    torch.cuda.synchronize()
    oracle.check_close(dw, oracle.grads_torch(x, w, None, dy, 1, 1)[1], acc_depth=8 * 28 * 28, what="tuned wgrad")


def test_on_miss_sweep_is_capped_checked_and_timed(tmp_path, monkeypatch, capsys):
    """An unrecorded shape through the operators with the default SPIO_TUNE=1: each family's
    sweep is capped (SPIO_TUNE_MAX_CONFIGS), every winner passed the cross-check against the
    family's any-shape kernel, results match the oracle, and the first-use cost is printed."""
    import time

    from spio_amd.functional import conv2d_gw8, reset_fused_backward_choices
    from spio_amd.kernels import conv2d_gw8_bgrad_kernel_factory
    from spio_amd.kernels.tuner import tuner as global_tuner

    db = tmp_path / "tune.json"
    monkeypatch.setenv("SPIO_TUNE_DB", str(db))
    monkeypatch.setenv("SPIO_TUNE", "1")
    monkeypatch.setenv("SPIO_TUNE_MAX_CONFIGS", "4")
    global_tuner._records.clear()  # the module-level tuner re-reads its record files
    for factory, kw in ((conv2d_gw8_kernel_factory, {}), (conv2d_gw8_kernel_factory, {"igrad": True}),
                        (conv2d_gw8_wgrad_kernel_factory, {}), (conv2d_gw8_bgrad_kernel_factory, {})):  # fmt: skip
        factory.get_kernel_cache(**kw).clear_cache()
    reset_fused_backward_choices()
    params = Conv2dGw8Params(n=6, c=88, h=36, w=30)  # in no record file
    x, w, _b, dy = oracle.make_args(params.n, params.c, params.h, params.w, 3, 3, 1, 1, False, 7)
    xg, wg, dyg = to_gpu(x), to_gpu(w), to_gpu(dy)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    y = conv2d_gw8(xg, wg, None, 1, 1, 1, 1, params.groups)
    torch.cuda.synchronize()
    t_fwd = time.perf_counter() - t0
    t0 = time.perf_counter()
    dx, dw, _ = torch.ops.spio.conv2d_gw8_backward(xg, wg, None, dyg, 1, 1, True, True, False)
    torch.cuda.synchronize()
    t_bwd = time.perf_counter() - t0
    with capsys.disabled():
        print(f"\nfirst use of an unrecorded shape with SPIO_TUNE_MAX_CONFIGS=4: forward {t_fwd:.2f} s, "
              f"backward (three families) {t_bwd:.2f} s")  # fmt: skip
    records = json.load(open(db))
    assert len(records) == 4  # fprop, dgrad, wgrad, bgrad
    assert all(rec["candidates"] <= 5 for rec in records.values())  # 4 ranked + the any-shape kernel
    oracle.check_close(y, oracle.fprop_torch(x, w, None, 1, 1), acc_depth=72, what="on-miss fprop")
    dx_e, dw_e, _ = oracle.grads_torch(x, w, None, dy, 1, 1)
    oracle.check_close(dx, dx_e, acc_depth=72, what="on-miss dgrad")
    oracle.check_close(dw, dw_e, acc_depth=params.n * params.p * params.q, what="on-miss wgrad")
    # second use: nothing is tuned or compiled again
    t0 = time.perf_counter()
    conv2d_gw8(xg, wg, None, 1, 1, 1, 1, params.groups)
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 0.05
    global_tuner._records.clear()
