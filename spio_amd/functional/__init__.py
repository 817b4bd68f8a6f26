"""Functional interface: the `spio::conv2d_gw8` custom operators."""

from .conv2d_gw8_function import (
    conv2d_gw8,
    conv2d_gw8_backward_op,
    fused_backward_kernel,
    reset_fused_backward_choices,
)
from .layernorm_2d_function import layernorm_2d
