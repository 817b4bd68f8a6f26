"""SPIO_LOGGER verbosity (reference: spio/util/logger.py:7-18)."""

import os

from .env import env_var_is_true

_raw = os.environ.get("SPIO_LOGGER", "0")
if _raw.isdigit():
    log_level = int(_raw)
elif env_var_is_true("SPIO_LOGGER"):
    log_level = 1
else:
    log_level = 0

logger_enabled = log_level > 0
logger_verbose = log_level > 1
