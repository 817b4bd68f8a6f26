"""Protocol of a layer-parameter object (reference: spio/kernels/params.py)."""

from typing import Protocol


class Params(Protocol):
    """Anything hashable that can name itself and check itself."""

    def encode(self) -> str:
        """A string usable inside a kernel name."""

    def validate(self) -> None:
        """Raise AssertionError when the parameters are not supported."""
