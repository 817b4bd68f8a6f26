"""Wall-clock timers gated by the logger level
(reference: spio/util/interval_timer.py:67-117)."""

import functools
import time

from .logger import logger_verbose


class Timer:
    """Context manager measuring elapsed wall-clock seconds."""

    def __init__(self, label: str = "", enabled: bool = True):
        self.label = label
        self.enabled = enabled
        self.seconds = 0.0

    def __enter__(self):
        self._start = time.perf_counter()
        return self

    def __exit__(self, *exc):
        self.seconds = time.perf_counter() - self._start
        if self.enabled and self.label:
            print(f"spio: {self.label} took {self.seconds * 1e3:.3f} ms")
        return False


def time_function(label: str = None, timer_class=Timer):
    """Decorator printing the duration of each call when SPIO_LOGGER > 1."""

    def decorate(fn):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            if not logger_verbose:
                return fn(*args, **kwargs)
            with timer_class(label or fn.__qualname__):
                return fn(*args, **kwargs)

        return wrapper

    return decorate
