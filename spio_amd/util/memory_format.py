"""Argument layout checks (reference: spio/util/memory_format.py:32-38)."""

import torch


def check_channels_last(args):
    """Assert that every 4-D tensor argument is channels_last contiguous."""
    for arg in args:
        if isinstance(arg, torch.Tensor) and arg.dim() == 4:
            assert arg.is_contiguous(
                memory_format=torch.channels_last
            ), f"Tensor is not channels_last: shape {tuple(arg.shape)} strides {arg.stride()}"
