"""Weight-gradient kernel family of conv2d_gw8.

Reference: spio/kernels/conv2d_gw8_wgrad_kernel.py:27-285.  The kernel adds
its partial sums into a pre-zeroed fp32 tensor laid out [K][R][S][8]
(spio/functional/conv2d_gw8_function.py:124-130).
"""

from dataclasses import dataclass
from typing import List

import torch

from ..util.math import divup
from .conv2d_gw8_kernel import _shape_defines
from .conv2d_gw8_params import Conv2dGw8Params
from .conv2d_stats import Conv2dStats
from .kernel import KernelSpec
from .kernel_factory import KernelFactory
from .launch_params import LaunchParams

DIRECT_SOURCE = "conv2d_gw8_direct.hip"


@dataclass(frozen=True)
class Conv2dGw8WgradConfig:
    """Tile configuration of the weight-gradient kernel.

    Attributes:
        groups: channel groups per workgroup.
        block_h: output rows per workgroup pass.
        block_n: images accumulated by one workgroup before its atomics.
        chunks: (direct variant) pixel chunks per group.
        variant: "mfma" or "direct".
    """

    groups: int = 8
    block_h: int = 8
    block_n: int = 1
    chunks: int = 64
    variant: str = "direct"


def _get_configs(params: Conv2dGw8Params, device_attr=None) -> List[Conv2dGw8WgradConfig]:
    num_cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    total_pix = params.n * params.p * params.q
    configs = []
    for mult in (4, 2, 8):
        chunks = max(1, min(divup(mult * num_cus, params.groups), divup(total_pix, 64)))
        cfg = Conv2dGw8WgradConfig(groups=1, block_h=1, block_n=1, chunks=chunks, variant="direct")
        if cfg not in configs:
            configs.append(cfg)
    return configs


def _get_kernel_spec(params: Conv2dGw8Params, config: Conv2dGw8WgradConfig, _device_attr=None) -> KernelSpec:
    params.validate()
    defines = _shape_defines(params)
    if config.variant == "direct":
        threads = 256
        defines.update(SPIO_WGRAD=1, SPIO_BLOCK_THREADS=threads, SPIO_WGRAD_CHUNKS=config.chunks)
        return KernelSpec(
            defines, LaunchParams(grid=params.groups * config.chunks, block=threads), DIRECT_SOURCE
        )
    raise ValueError(f"unknown kernel variant {config.variant!r}")


def _make_test_args(params: Conv2dGw8Params, device):
    """Synthetic (grad_weight, x, dy) for timing."""
    cl = torch.channels_last
    x = torch.randn(params.input_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dy = torch.randn(params.output_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dw = torch.zeros(params.weight_shape, device=device, dtype=torch.float32).contiguous(memory_format=cl)
    return (dw, x, dy)


conv2d_gw8_wgrad_kernel_factory = KernelFactory(
    Conv2dGw8Params,
    Conv2dGw8WgradConfig,
    Conv2dStats,
    kernel_name="spio_conv2d_gw8_wgrad",
    configs=_get_configs,
    kernel_spec=_get_kernel_spec,
    make_test_args=_make_test_args,
)
