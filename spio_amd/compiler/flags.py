"""Compiler settings read from the environment.

Same switches as the reference (spio/compiler/flags.py:10-19): SPIO_WORKERS,
SPIO_LINEINFO, SPIO_DEBUG; SPIO_CODE_CACHE (default on) controls the on-disk
cache of compiled code objects.
"""

import os
from contextvars import ContextVar

from ..util.env import env_var_is_true

DEFAULT_WORKERS = 4

workers = max(1, int(os.environ.get("SPIO_WORKERS", str(DEFAULT_WORKERS))))
lineinfo = ContextVar("lineinfo", default=env_var_is_true("SPIO_LINEINFO"))
debug = ContextVar("debug", default=env_var_is_true("SPIO_DEBUG"))
code_cache_enabled = ContextVar(
    "code_cache_enabled", default=env_var_is_true("SPIO_CODE_CACHE", default="True")
)
