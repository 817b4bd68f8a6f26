"""Environment-variable parsing (reference: spio/util/env.py:8-20)."""

import os

_TRUE_WORDS = ("true", "yes", "y", "t")


def env_var_is_true(env_var: str, default: str = "False") -> bool:
    """True for y/yes/t/true (any case) and for positive integers."""
    value = os.environ.get(env_var, default).strip().lower()
    if value in _TRUE_WORDS:
        return True
    if value.isdigit():
        return int(value) > 0
    return False
