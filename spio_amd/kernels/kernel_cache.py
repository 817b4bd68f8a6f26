"""Per-kernel cache of loaded kernels keyed by (device, params).

Reference: spio/kernels/kernel_cache.py:21-111, including the overlay used to
pin configurations while benchmarking.  A cache miss asks the tuner for the
best configuration (the reference asks its XGBoost model), compiles and loads
it.  A lock makes get() safe from several threads.
"""

import threading
from typing import Dict

import torch

from ..compiler.compiler_pool import compile_kernel_configs
from ..hip.driver import get_device_attributes
from ..util.logger import logger_enabled
from .kernel import Kernel
from .kernel_key import KernelKey
from .kernel_params_logger import kernel_params_logging_is_enabled, log_kernel_params
from .tuner import tuner


def _ordinal(device) -> int:
    idx = torch.device(device).index
    return torch.cuda.current_device() if idx is None else idx


class KernelCache:
    """Cache of compiled and loaded kernels for one kernel name."""

    def __init__(self):
        self._cache: Dict[KernelKey, Kernel] = {}
        self._cache_overlay: Dict[KernelKey, Kernel] = {}
        self._lock = threading.RLock()

    def update_overlay(self, overlay: Dict[KernelKey, Kernel]):
        """Kernels that take precedence over (and hide) the main cache."""
        with self._lock:
            self._cache_overlay.update(overlay)

    def clear_overlay(self):
        with self._lock:
            self._cache_overlay.clear()

    def clear_cache(self):
        with self._lock:
            self._cache.clear()

    @log_kernel_params
    def get(self, kernel_factory, params, device, **kernel_kwargs) -> Kernel:
        """The kernel to run for `params` on `device`; compiles on first use."""
        ordinal = _ordinal(device)
        key = KernelKey(device_ordinal=ordinal, params=params)
        with self._lock:
            kernel = self._cache_overlay.get(key)
            if kernel is not None:
                return kernel
            if self._cache_overlay:
                raise ValueError(
                    f"Kernel {kernel_factory} with params {params} and device {device} "
                    f"not found in overlay cache"
                )
            kernel = self._cache.get(key)
            if kernel is not None:
                return kernel
            device_attr = get_device_attributes(ordinal)
            if kernel_params_logging_is_enabled():
                config = next(iter(kernel_factory.configs(params, device_attr, **kernel_kwargs)))
                kernel = compile_and_load_kernel(
                    kernel_factory, params, config, ordinal, device_attr, **kernel_kwargs
                )
            else:
                kernel = tuner.best_kernel(
                    kernel_factory, params, ordinal, device_attr, **kernel_kwargs
                )
            self._cache[key] = kernel
            if logger_enabled:
                print(f"spio: compiled kernel {kernel} for device {device}.")
            return kernel


def compile_and_load_kernel(kernel_factory, params, config, ordinal, device_attr, **kernel_kwargs):
    """Compile one configuration and load it on device `ordinal`."""
    kernels = compile_kernel_configs(
        kernel_factory, params, configs=[config], device_attr=device_attr, **kernel_kwargs
    )
    kernels[0].load(device_ordinal=ordinal)
    return kernels[0]
