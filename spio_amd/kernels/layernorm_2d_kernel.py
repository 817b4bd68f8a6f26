"""LayerNorm over the channels of an NHWC fp16 tensor: parameters, configurations, factory.

The reference ships the device source of such a kernel (spio/src/layernorm_2d.cu:81-222: NHWC
fp16 in and out, fp32 mean and variance over C per pixel, optional fp32 weight and bias) without
a Python side; this module gives the re-designed kernel (csrc/layernorm_2d.hip) the same
factory / cache / tuner plumbing as the convolution kernels.

Kernel arguments: (output, input, weight or None, bias or None).
"""

import re
from dataclasses import dataclass
from typing import List

import torch

from ..util.math import divup
from .kernel import KernelSpec
from .kernel_factory import KernelFactory
from .launch_params import LaunchParams

SOURCE = "layernorm_2d.hip"


@dataclass(frozen=True)
class LayerNorm2dParams:
    """Shape of one channel LayerNorm: input [n, c, h, w] with channels_last strides."""

    n: int
    c: int
    h: int
    w: int
    eps: float = 1e-6
    has_weight: bool = True
    has_bias: bool = True

    def encode(self) -> str:
        """The name is part of the kernel's symbol, so it holds identifier characters only: eps is
        its shortest round-trip decimal form with '.' written 'p', '-' written 'm' and '+' dropped
        (1e-06 -> 1em06, 0.001 -> 0p001, 1.5e-05 -> 1p5em05)."""
        flags = ("w" if self.has_weight else "nw") + ("b" if self.has_bias else "nb")
        eps = repr(float(self.eps)).replace(".", "p").replace("-", "m").replace("+", "")
        return f"{self.n}n_{self.c}c_{self.h}h_{self.w}w_{eps}eps_{flags}"

    _PATTERN = re.compile(r"(\d+)n_(\d+)c_(\d+)h_(\d+)w_([0-9epm]+)eps_(w|nw)(b|nb)$")

    @classmethod
    def decode(cls, string: str) -> "LayerNorm2dParams":
        m = cls._PATTERN.match(string)
        if m is None:
            raise ValueError("Invalid string representation.")
        n, c, h, w = (int(v) for v in m.groups()[:4])
        return cls(n=n, c=c, h=h, w=w, eps=float(m.group(5).replace("p", ".").replace("m", "-")),
                   has_weight=m.group(6) == "w", has_bias=m.group(7) == "b")  # fmt: skip

    def validate(self):
        assert self.n > 0 and self.h > 0 and self.w > 0
        assert self.c > 0 and self.c % 8 == 0, "channels must be a multiple of 8 (16-byte units)"
        assert self.c <= 8 * 64 * 4, "at most 2048 channels"
        assert self.eps > 0

    @property
    def pixels(self) -> int:
        return self.n * self.h * self.w

    @property
    def shape(self):
        return (self.n, self.c, self.h, self.w)


@dataclass(frozen=True)
class LayerNorm2dConfig:
    """threads per workgroup, pixel groups in flight per lane, workgroups per compute unit, and
    the lanes that share a pixel (0: the smallest power of two that gives every 16-byte unit of a
    pixel its own lane; a smaller power of two gives each lane several units, which keeps all
    lanes busy when C/8 is not a power of two: 96 channels = 12 units = 4 lanes x 3 units)."""

    threads: int = 256
    unroll: int = 4
    groups_per_cu: int = 8
    lanes: int = 0


def lanes_per_pixel(c: int) -> int:
    units = c // 8
    lpp = 1
    while lpp < units and lpp < 64:
        lpp *= 2
    return lpp


def _lane_choices(c: int) -> List[int]:
    """Lanes per pixel worth trying: the default, and where that leaves lanes idle the largest
    power of two that divides the units of a pixel (at most 4 units per lane)."""
    units = c // 8
    full = lanes_per_pixel(c)
    out = [0]
    if full != units:
        exact = units & -units  # largest power of two dividing units
        if exact < full and divup(units, exact) <= 4:
            out.append(exact)
    return out


def _get_configs(params: LayerNorm2dParams, _device_attr=None) -> List[LayerNorm2dConfig]:
    per_lanes = []
    for lanes in _lane_choices(params.c):
        upl = divup(params.c // 8, lanes or lanes_per_pixel(params.c))
        mine = []
        for threads in (256, 512):
            for unroll in (8, 4, 2, 1):  # as many loads in flight as the registers hold
                if unroll * upl > 8:
                    continue
                for per_cu in (8, 16, 4):
                    mine.append(LayerNorm2dConfig(threads, unroll, per_cu, lanes))
        per_lanes.append(mine)
    # the lane choices alternate, busy lanes first, so that a sweep cut short has seen both
    out = []
    for i in range(max(len(m) for m in per_lanes)):
        for mine in reversed(per_lanes):
            if i < len(mine):
                out.append(mine[i])
    return out or [LayerNorm2dConfig(256, 1, 8)]


def _get_kernel_spec(params: LayerNorm2dParams, config: LayerNorm2dConfig, device_attr=None) -> KernelSpec:
    params.validate()
    cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    lpp = config.lanes or lanes_per_pixel(params.c)
    assert lpp & (lpp - 1) == 0 and lpp <= 64 and divup(params.c // 8, lpp) <= 4, f"illegal configuration {config}"
    pass_pixels = (64 // lpp) * (config.threads // 64) * config.unroll
    grid = max(1, min(divup(params.pixels, pass_pixels), cus * config.groups_per_cu))
    defines = {
        "SPIO_LN_C": params.c, "SPIO_LN_PIXELS": params.pixels, "SPIO_LN_LPP": lpp,
        "SPIO_LN_THREADS": config.threads, "SPIO_LN_UNROLL": config.unroll,
        "SPIO_LN_HAS_WEIGHT": int(params.has_weight), "SPIO_LN_HAS_BIAS": int(params.has_bias),
        "SPIO_LN_EPS": f"{float(params.eps)!r}f", "SPIO_LN_GRID": grid,
    }  # fmt: skip
    return KernelSpec(defines, LaunchParams(grid=grid, block=config.threads), SOURCE,
                      notes={"LPP": lpp, "PASS_PIXELS": pass_pixels})  # fmt: skip


def _make_test_args(params: LayerNorm2dParams, device):
    cl = torch.channels_last
    x = torch.randn(params.shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    y = torch.empty_like(x)
    w = torch.randn(params.c, device=device, dtype=torch.float32) if params.has_weight else None
    b = torch.randn(params.c, device=device, dtype=torch.float32) if params.has_bias else None
    return (y, x, w, b)


layernorm_2d_kernel_factory = KernelFactory(
    LayerNorm2dParams,
    LayerNorm2dConfig,
    None,
    kernel_name="spio_layernorm_2d",
    configs=_get_configs,
    kernel_spec=_get_kernel_spec,
    make_test_args=_make_test_args,
)


# ---- backward: grad_input and per-workgroup partial sums of grad_weight / grad_bias ----
#
# Kernel arguments: (sums, grad_input, input, grad_output, weight or None); `sums` is fp32 [2][C]
# (0 = grad_weight, 1 = grad_bias) and is overwritten.  Two stages: the main kernel writes one row
# of partial sums per workgroup into a workspace of [grid][2][C] floats, the <name>_reduce kernel
# adds the rows.

BWD_SOURCE = "layernorm_2d_bwd.hip"
BWD_MAX_CHANNELS = 1024  # the workgroup's channel sums meet in LDS: waves x 2 x C floats
BWD_MAX_GROUPS_PER_CU = 4


@dataclass(frozen=True)
class LayerNorm2dBwdConfig:
    """As LayerNorm2dConfig; `unroll` counts pixel groups whose input and grad_output loads are
    in flight together, and few workgroups per compute unit keep the partial sums few."""

    threads: int = 256
    unroll: int = 2
    groups_per_cu: int = 2
    lanes: int = 0


def layernorm_2d_bwd_is_supported(params: LayerNorm2dParams) -> bool:
    return params.c % 8 == 0 and params.c <= BWD_MAX_CHANNELS


def _get_bwd_configs(params: LayerNorm2dParams, _device_attr=None) -> List[LayerNorm2dBwdConfig]:
    if not layernorm_2d_bwd_is_supported(params):
        return []
    per_lanes = []
    for lanes in _lane_choices(params.c):
        upl = divup(params.c // 8, lanes or lanes_per_pixel(params.c))
        mine = []
        for threads in (256, 512):
            for unroll in (4, 2, 1):
                if unroll * upl > 4:
                    continue
                for per_cu in (2, 4, 1):
                    mine.append(LayerNorm2dBwdConfig(threads, unroll, per_cu, lanes))
        per_lanes.append(mine)
    out = []
    for i in range(max(len(m) for m in per_lanes)):
        for mine in reversed(per_lanes):
            if i < len(mine):
                out.append(mine[i])
    return out


def _get_bwd_kernel_spec(params: LayerNorm2dParams, config: LayerNorm2dBwdConfig, device_attr=None) -> KernelSpec:
    params.validate()
    assert layernorm_2d_bwd_is_supported(params), f"unsupported shape {params}"
    cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    lpp = config.lanes or lanes_per_pixel(params.c)
    assert lpp & (lpp - 1) == 0 and lpp <= 64 and divup(params.c // 8, lpp) <= 4, f"illegal configuration {config}"
    assert 1 <= config.groups_per_cu <= BWD_MAX_GROUPS_PER_CU
    pass_pixels = (64 // lpp) * (config.threads // 64) * config.unroll
    grid = max(1, min(divup(params.pixels, pass_pixels), cus * config.groups_per_cu))
    defines = {
        "SPIO_LN_C": params.c, "SPIO_LN_PIXELS": params.pixels, "SPIO_LN_LPP": lpp,
        "SPIO_LN_THREADS": config.threads, "SPIO_LN_UNROLL": config.unroll,
        "SPIO_LN_HAS_WEIGHT": int(params.has_weight),
        "SPIO_LN_EPS": f"{float(params.eps)!r}f", "SPIO_LN_GRID": grid,
    }  # fmt: skip
    spec = KernelSpec(defines, LaunchParams(grid=grid, block=config.threads), BWD_SOURCE,
                      notes={"LPP": lpp, "PASS_PIXELS": pass_pixels, "GRID": grid})  # fmt: skip
    spec.workspace_bytes = grid * 2 * params.c * 4
    spec.epilogue_suffix = "_reduce"
    spec.epilogue_launch_params = LaunchParams(grid=divup(2 * params.c, 32), block=256)
    return spec


def _make_bwd_test_args(params: LayerNorm2dParams, device):
    cl = torch.channels_last
    x = torch.randn(params.shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dy = torch.randn(params.shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dx = torch.empty_like(x)
    w = torch.randn(params.c, device=device, dtype=torch.float32) if params.has_weight else None
    sums = torch.empty((2, params.c), device=device, dtype=torch.float32)
    return (sums, dx, x, dy, w)


layernorm_2d_bwd_kernel_factory = KernelFactory(
    LayerNorm2dParams,
    LayerNorm2dBwdConfig,
    None,
    kernel_name="spio_layernorm_2d_bwd",
    configs=_get_bwd_configs,
    kernel_spec=_get_bwd_kernel_spec,
    make_test_args=_make_bwd_test_args,
)

