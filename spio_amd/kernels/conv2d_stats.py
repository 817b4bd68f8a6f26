"""Algorithmic bytes / MACs / accumulation depth of conv2d_gw8.

Restates spio/kernels/conv2d_stats.py:8-126.  The byte counts are the
"algorithmic bytes" behind every effective-bandwidth figure: each tensor
crosses HBM once.  The reference counts grad_weight at `unit` bytes per
element although the kernel writes fp32; `grad_weight_bytes_written_fp32`
gives the figure with 4-byte elements.
"""

from math import prod

from .stats import Stats


class Conv2dStats(Stats):
    """Statistics for one Conv2dGw8Params."""

    # element counts
    @property
    def _nx(self) -> int:
        return prod(self.params.input_shape)

    @property
    def _ny(self) -> int:
        return prod(self.params.output_shape)

    @property
    def _nw(self) -> int:
        return prod(self.params.weight_shape)

    @property
    def _nb(self) -> int:
        return prod(self.params.bias_shape) if self.params.has_bias else 0

    @property
    def _depth(self) -> int:
        """Products summed per output element: R * S * group width."""
        return self.params.r * self.params.s * self.params.group_width

    # forward
    @property
    def output_macs(self):
        """An added bias counts as half a MAC per output element."""
        return self._ny * self._depth + (self._ny / 2 if self.params.has_bias else 0)

    @property
    def output_bytes_read(self) -> int:
        return (self._nx + self._nw + self._nb) * self.unit

    @property
    def output_bytes_written(self) -> int:
        return self._ny * self.unit

    @property
    def output_accumulation_depth(self) -> int:
        return self._depth

    # data gradient
    @property
    def grad_input_macs(self):
        return self._nx * self._depth

    @property
    def grad_input_bytes_read(self) -> int:
        return (self._ny + self._nw) * self.unit

    @property
    def grad_input_bytes_written(self) -> int:
        return self._nx * self.unit

    @property
    def grad_input_accumulation_depth(self) -> int:
        return self._depth

    # weight gradient
    @property
    def grad_weight_macs(self):
        return self._nx * self._depth

    @property
    def grad_weight_bytes_read(self) -> int:
        return (self._ny + self._nx) * self.unit

    @property
    def grad_weight_bytes_written(self) -> int:
        return self._nw * self.unit

    @property
    def grad_weight_bytes_written_fp32(self) -> int:
        return self._nw * 4

    @property
    def grad_weight_accumulation_depth(self) -> int:
        return self.params.n * self.params.h * self.params.w

    # bias gradient
    @property
    def grad_bias_macs(self):
        return self._ny / 2

    @property
    def grad_bias_bytes_read(self) -> int:
        return self._ny * self.unit

    @property
    def grad_bias_bytes_written(self) -> int:
        return self._nb * self.unit

    @property
    def grad_bias_accumulation_depth(self) -> int:
        return self.params.n * self.params.h * self.params.w
