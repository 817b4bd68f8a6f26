"""Factory tying a params class, a configuration space and a kernel source together.

Reference: spio/kernels/kernel_factory.py:79-216.  Keyword arguments
(`igrad=True`) select between modes of one kernel family; each mode has its
own name and its own cache.
"""

from typing import Any, Callable, Dict, Iterable, Union

from ..util.memory_format import check_channels_last
from .kernel import Kernel, KernelSpec, get_full_kernel_name
from .kernel_cache import KernelCache


class KernelFactory:
    """Creates Kernel objects and hands out the best one per (params, device)."""

    def __init__(
        self,
        params_cls=None,
        config_cls=None,
        stats_cls=None,
        kernel_name: Union[str, Callable[..., str]] = None,
        configs: Union[Iterable[Any], Callable[..., Iterable[Any]]] = None,
        kernel_spec: Union[KernelSpec, Callable[..., KernelSpec]] = None,
        make_test_args: Callable[..., Any] = None,
        args_checker=check_channels_last,
    ):
        self.params_cls = params_cls
        self.config_cls = config_cls
        self.stats_cls = stats_cls
        self._kernel_name = kernel_name
        self._configs = configs
        self._kernel_spec = kernel_spec
        self._make_test_args = make_test_args
        self._args_checker = args_checker
        self._kernel_caches: Dict[str, KernelCache] = {}

    def configs(self, params, device_attr=None, **kwargs):
        """All legal configurations for `params`, most promising first."""
        if callable(self._configs):
            return self._configs(params, device_attr, **kwargs)
        return self._configs

    def get_kernel_name(self, **kwargs) -> str:
        if callable(self._kernel_name):
            return self._kernel_name(**kwargs)
        return self._kernel_name

    def get_full_kernel_name(self, params, **kwargs) -> str:
        return get_full_kernel_name(self.get_kernel_name(**kwargs), params)

    def get_kernel_spec(self, params, config, device_attr=None, **kwargs) -> KernelSpec:
        if callable(self._kernel_spec):
            return self._kernel_spec(params, config, device_attr, **kwargs)
        return self._kernel_spec

    def get_kernel_cache(self, **kwargs) -> KernelCache:
        name = self.get_kernel_name(**kwargs)
        cache = self._kernel_caches.get(name)
        if cache is None:
            cache = self._kernel_caches.setdefault(name, KernelCache())
        return cache

    def get_kernel(self, params, device, **kwargs) -> Kernel:
        """Cached best kernel for the params on the device (tunes/compiles on a miss)."""
        return self.get_kernel_cache(**kwargs).get(self, params, device, **kwargs)

    def make_kernel(self, params, config, device_attr=None, **kwargs) -> Kernel:
        """A new, not yet compiled Kernel for one configuration."""
        return Kernel(
            self.get_full_kernel_name(params, **kwargs),
            self.get_kernel_spec(params, config, device_attr, **kwargs),
            params=params,
            config=config,
            args_checker=self._args_checker,
        )

    def make_test_args(self, params, device, **kwargs):
        """Synthetic launch arguments for timing a kernel of this family."""
        if self._make_test_args is None:
            raise ValueError("this kernel family does not define synthetic arguments")
        return self._make_test_args(params, device, **kwargs)

    def __repr__(self):
        return f"KernelFactory({self._kernel_name})"
