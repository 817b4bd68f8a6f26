"""Records which kernels a model asks for (reference: spio/kernels/kernel_params_logger.py:22-111).

    with KernelParamsLogger() as logger:
        model(x).sum().backward()
    for kp in logger.get_logged_params(): ...

While a logger is active the kernel cache does not tune: it takes the first
configuration, as the reference does (spio/kernels/kernel_cache.py:71-81).
"""

import functools
import threading
from contextlib import ContextDecorator
from typing import List, Optional

from .kernel_key import KernelParams

_active: Optional["KernelParamsLogger"] = None
_active_lock = threading.Lock()


class KernelParamsLogger(ContextDecorator):
    """Context manager collecting KernelParams of every KernelCache.get call."""

    def __init__(self):
        self.logged_params: List[KernelParams] = []
        self._lock = threading.Lock()

    def __enter__(self):
        global _active
        with _active_lock:
            _active = self
        self.logged_params = []
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        global _active
        with _active_lock:
            _active = None
        return False

    def get_logged_params(self) -> List[KernelParams]:
        """Requests seen so far, in call order."""
        return self.logged_params

    def record(self, kernel_cache, kernel_factory, params, device, **kernel_kwargs):
        """Append one request (thread-safe)."""
        with self._lock:
            self.logged_params.append(
                KernelParams(kernel_cache, kernel_factory, params, device, tuple(kernel_kwargs.items()))
            )


def get_global_logger() -> Optional[KernelParamsLogger]:
    """The active logger, if any."""
    with _active_lock:
        return _active


def kernel_params_logging_is_enabled() -> bool:
    """True inside a `with KernelParamsLogger()` block."""
    return get_global_logger() is not None


def log_kernel_params(method):
    """Decorator for KernelCache.get(self, kernel_factory, params, device, **kwargs)."""

    @functools.wraps(method)
    def wrapper(self, kernel_factory, params, device, **kwargs):
        logger = get_global_logger()
        if logger is not None:
            logger.record(self, kernel_factory, params, device, **kwargs)
        return method(self, kernel_factory, params, device, **kwargs)

    return wrapper
