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
