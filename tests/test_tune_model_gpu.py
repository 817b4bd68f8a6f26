"""In-situ tuning: the params logger records the kernels a model asks for, `tune_model` times
their candidate configurations inside the model through the caches' overlays, records the
winners, and the model then runs with them and still matches the CPU oracle.
(Reference procedure: scripts/profile_block.py:545-701, spio/kernels/kernel_cache.py:34-47,71-81,
spio/kernels/kernel_params_logger.py:22-111.)"""

import json

import pytest
import torch
from torch import nn

from helpers import to_gpu
from oracle import conv2d_gw8_oracle as oracle
from spio_amd.functional import conv2d_gw8
from spio_amd.hip import get_device_attributes
from spio_amd.kernels import (
    Conv2dGw8Params,
    KernelKey,
    KernelParamsLogger,
    conv2d_gw8_kernel_factory,
)
from spio_amd.kernels.kernel import LaunchTimer
from spio_amd.layers import Conv2dGw8
from spio_amd.tune import tune_model

pytestmark = pytest.mark.gpu


class TwoConvs(nn.Module):
    def __init__(self):
        super().__init__()
        self.a = Conv2dGw8(64, 64, 3, padding=1, groups=8)
        self.b = Conv2dGw8(64, 64, 5, padding=2, groups=8, bias=False)

    def forward(self, x):
        return self.b(torch.relu(self.a(x)))


def _cpu_reference(model, x):
    xa = x.half().float()
    ya = oracle.fprop_torch(xa.half(), model.a.weight.detach().cpu().half(), model.a.bias.detach().cpu().float(), 1, 1)
    ya = torch.relu(ya.half().float())
    return oracle.fprop_torch(ya.half(), model.b.weight.detach().cpu().half(), None, 2, 2)


def test_logger_sees_the_three_families():
    torch.manual_seed(0)
    model = TwoConvs().cuda().to(memory_format=torch.channels_last)
    x = torch.randn(4, 64, 20, 20, device="cuda").contiguous(memory_format=torch.channels_last).requires_grad_(True)
    with KernelParamsLogger() as logger:
        with torch.autocast(device_type="cuda", dtype=torch.float16):
            model(x).float().sum().backward()
    names = {kp.kernel_factory.get_kernel_name(**dict(kp.kernel_kwargs)) for kp in logger.get_logged_params()}
    assert {"spio_conv2d_gw8_fprop", "spio_conv2d_gw8_dgrad", "spio_conv2d_gw8_wgrad"} <= names
    shapes = {kp.params.encode() for kp in logger.get_logged_params()}
    assert shapes == {"4n_64c_20h_20w_1py_1px_3r_3s_b", "4n_64c_20h_20w_2py_2px_5r_5s_nb"}


def test_overlay_pins_the_configuration_that_is_launched():
    attr = get_device_attributes(0)
    params = Conv2dGw8Params(n=2, c=64, h=20, w=20, padding=(1, 1))  # as the operator builds it
    configs = list(conv2d_gw8_kernel_factory.configs(params, attr))
    kernel = conv2d_gw8_kernel_factory.make_kernel(params, configs[3], attr)
    kernel.compile()
    kernel.load(0)
    cache = conv2d_gw8_kernel_factory.get_kernel_cache()
    x, w, _b, _dy = oracle.make_args(2, 64, 20, 20, 3, 3, 1, 1, False, 5)
    cache.update_overlay({KernelKey(device_ordinal=0, params=params): kernel})
    try:
        with LaunchTimer() as timer:
            y = conv2d_gw8(to_gpu(x), to_gpu(w), None, 1, 1, 1, 1, 8)
            averages = timer.averages()
    finally:
        cache.clear_overlay()
    assert list(averages) == [kernel] and averages[kernel] > 0
    oracle.check_close(y, oracle.fprop_torch(x, w, None, 1, 1), acc_depth=72, what="pinned configuration")
    kernel.unload()


def test_tune_model_records_winners_and_model_still_matches(tmp_path, monkeypatch):
    db = tmp_path / "tuned.json"
    monkeypatch.setenv("SPIO_TUNE_DB", str(db))
    monkeypatch.setenv("SPIO_TUNE", "1")
    torch.manual_seed(1)
    model = TwoConvs().cuda().to(memory_format=torch.channels_last)
    xs = [torch.randn(4, 64, 20, 20, device="cuda").contiguous(memory_format=torch.channels_last).requires_grad_(True)
          for _ in range(2)]  # fmt: skip
    results = tune_model(model, xs, backward=True, max_configs=3, iters=2, warmup=1,
                         autocast_dtype=torch.float16, record_path=str(db))  # fmt: skip
    by_name = {r["kernel"]: r for r in results}
    for shape in ("4n_64c_20h_20w_1py_1px_3r_3s_b", "4n_64c_20h_20w_2py_2px_5r_5s_nb"):
        for family in ("fprop", "dgrad", "wgrad", "bgrad"):
            entry = by_name[f"spio_conv2d_gw8_{family}__{shape}"]
            assert entry["config"] is not None and entry["us"] > 0, entry
            assert 1 <= len(entry["sweep"]) <= 3
    records = json.load(open(db))
    assert all(rec.get("in_situ") for rec in records.values()) and len(records) == len(results)
    # the model now runs with the recorded winners and still computes the right thing
    model.zero_grad()
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.float16):
        got = model(xs[0])
    want = _cpu_reference(model, xs[0].detach().cpu())
    oracle.check_close(got, want, rtol=4e-3, atol=2e-2, what="model after in-situ tuning")
