"""Compile many kernels concurrently.

The reference uses a process pool created at import
(spio/compiler/compiler_pool.py:19-86).  hipRTC runs inside the calling
process and ctypes releases the GIL around it, so a lazily created thread pool
gives the same overlap without forking a process that may hold a GPU context.
"""

import threading
from concurrent.futures import ThreadPoolExecutor
from typing import Any, List, Optional

from . import flags

_pool: Optional[ThreadPoolExecutor] = None
_pool_lock = threading.Lock()


def _get_pool() -> ThreadPoolExecutor:
    global _pool
    with _pool_lock:
        if _pool is None:
            _pool = ThreadPoolExecutor(max_workers=flags.workers, thread_name_prefix="spio-hiprtc")
        return _pool


def compile_kernels(kernels: List[Any]) -> None:
    """Compile every Kernel in the list (sets kernel.code)."""
    if len(kernels) <= 1 or flags.workers <= 1:
        for kernel in kernels:
            kernel.compile()
        return
    futures = [_get_pool().submit(kernel.compile) for kernel in kernels]
    errors = []
    for f in futures:
        try:
            f.result()
        except Exception as e:  # pylint: disable=broad-except
            errors.append(e)
    if errors:
        raise ValueError(f"Error compiling kernels: {errors[0]}") from errors[0]


def compile_kernel_configs(
    kernel_factory, params, configs: Optional[List[Any]] = None, device_attr=None, **kernel_kwargs
) -> List[Any]:
    """Make and compile one Kernel per configuration (all configurations by default)."""
    if configs is None:
        configs = list(kernel_factory.configs(params, device_attr, **kernel_kwargs))
    kernels = [
        kernel_factory.make_kernel(params, config=config, device_attr=device_attr, **kernel_kwargs)
        for config in configs
    ]
    compile_kernels(kernels)
    return kernels
