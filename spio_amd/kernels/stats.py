"""Byte and MAC accounting shared by all kernels (reference: spio/kernels/stats.py:8-67)."""

from typing import List, Union


class Stats:
    """Totals over the tensors named in `output_names`.

    Subclasses provide `<name>_macs`, `<name>_bytes_read`,
    `<name>_bytes_written` and `<name>_accumulation_depth` for each output
    name ('output', 'grad_input', 'grad_weight', 'grad_bias').
    """

    def __init__(self, params=None, unit: int = 2, output_names: Union[str, List[str]] = None):
        self.params = params
        self.unit = unit
        if isinstance(output_names, str):
            output_names = [output_names]
        self.output_names = list(output_names or [])

    def _total(self, suffix: str):
        return sum(getattr(self, f"{name}_{suffix}") for name in self.output_names)

    @property
    def macs(self):
        return self._total("macs")

    @property
    def bytes_read(self) -> int:
        return self._total("bytes_read")

    @property
    def bytes_written(self) -> int:
        return self._total("bytes_written")

    @property
    def bytes(self) -> int:
        return self.bytes_read + self.bytes_written

    @property
    def op_byte(self) -> float:
        """Floating-point operations (2 per MAC) per byte moved."""
        return 2.0 * self.macs / self.bytes

    @property
    def accumulation_depths(self) -> List[int]:
        return [getattr(self, f"{name}_accumulation_depth") for name in self.output_names]
