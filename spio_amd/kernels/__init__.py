"""Kernel families, parameters, statistics and the kernel cache."""

from .conv2d_gw8_params import Conv2dGw8Params
from .conv2d_stats import Conv2dStats
from .stats import Stats
from .params import Params
from .launch_params import LaunchParams
from .kernel_key import KernelKey, KernelParams
from .kernel import Kernel, KernelSpec, get_full_kernel_name
from .kernel_factory import KernelFactory
from .kernel_cache import KernelCache
from .kernel_params_logger import KernelParamsLogger, kernel_params_logging_is_enabled
from .tuner import tuner, Tuner
from .conv2d_gw8_kernel import conv2d_gw8_kernel_factory, Conv2dGw8Config
from .conv2d_gw8_wgrad_kernel import conv2d_gw8_wgrad_kernel_factory, Conv2dGw8WgradConfig
from .conv2d_gw8_bgrad_kernel import (
    conv2d_gw8_bgrad_kernel_factory,
    Conv2dGw8BgradConfig,
    bgrad_is_supported,
)
from .layernorm_2d_kernel import (
    layernorm_2d_kernel_factory,
    layernorm_2d_bwd_kernel_factory,
    layernorm_2d_bwd_is_supported,
    LayerNorm2dParams,
    LayerNorm2dConfig,
    LayerNorm2dBwdConfig,
)
