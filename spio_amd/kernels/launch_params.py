"""Grid / block / dynamic-LDS of one launch (reference: spio/kernels/launch_params.py:7-39)."""

from dataclasses import dataclass
from typing import Tuple, Union


def _as_3_tuple(value) -> Tuple[int, int, int]:
    if isinstance(value, int):
        value = (value,)
    value = tuple(int(v) for v in value)
    if not 1 <= len(value) <= 3:
        raise ValueError("Value must be an int or a tuple of at most 3 integers.")
    for v in value:
        assert v > 0, "All launch dimensions must be positive."
    return value + (1,) * (3 - len(value))


@dataclass
class LaunchParams:
    """Launch geometry, normalised to 3-tuples."""

    grid: Union[int, Tuple[int, ...]]
    block: Union[int, Tuple[int, ...]]
    shared_mem_bytes: int = 0

    def __post_init__(self):
        self.grid = _as_3_tuple(self.grid)
        self.block = _as_3_tuple(self.block)
