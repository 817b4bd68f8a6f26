"""`Conv2dGw8`: an nn.Conv2d whose forward runs spio::conv2d_gw8.

Reference: spio/layers/conv2d_gw8.py:12-139.  Parameters stay fp32; under
torch.autocast the operator casts them to fp16 (bias stays fp32).
"""

from typing import Optional, Tuple

import torch
from torch import nn

from ..functional import conv2d_gw8
from ..kernels import Conv2dGw8Params


def _pair(x) -> Tuple[int, int]:
    return (x, x) if isinstance(x, int) else tuple(x)


class Conv2dGw8(nn.Conv2d):
    """Grouped conv2d with group width 8 (C_in == C_out, groups == C // 8)."""

    Params = Conv2dGw8Params

    @staticmethod
    def make(*args, **kwargs) -> Optional[nn.Module]:
        """A Conv2dGw8 when the nn.Conv2d arguments qualify, else None.

        Positional arguments follow `match_args`, whose order
        (in, out, kernel_size, stride, dilation, groups) differs from
        nn.Conv2d's after `stride` (reference: conv2d_gw8.py:27-42, 61-70);
        pass everything after kernel_size by keyword.
        """
        if Conv2dGw8.match_args(*args, **kwargs):
            return Conv2dGw8(*args, **kwargs)
        return None

    @staticmethod
    def match(module: nn.Module) -> bool:
        """True for a plain nn.Conv2d that this layer can replace."""
        return (
            isinstance(module, nn.Conv2d)
            and not isinstance(module, Conv2dGw8)
            and isinstance(module.padding, (tuple, list, int))
            and Conv2dGw8.match_args(
                module.in_channels, module.out_channels, module.kernel_size,
                module.stride, module.dilation, module.groups,
                padding_mode=module.padding_mode,
            )  # fmt: skip
        )

    @staticmethod
    def match_args(in_channels, out_channels, kernel_size, stride=1, dilation=1, groups=1,
                   padding_mode="zeros", **_kwargs) -> bool:  # fmt: skip
        """The matching rule of the reference (conv2d_gw8.py:61-90): kernel sizes 1..5."""
        r, s = _pair(kernel_size)
        return (
            in_channels == out_channels
            and groups > 0
            and in_channels // groups == 8
            and in_channels % groups == 0
            and 1 <= r <= 5
            and 1 <= s <= 5
            and _pair(dilation) == (1, 1)
            and _pair(stride) == (1, 1)
            and padding_mode == "zeros"
        )

    @staticmethod
    def from_torch_module(conv2d: nn.Conv2d) -> "Conv2dGw8":
        """A Conv2dGw8 sharing (not copying) the parameters of `conv2d`."""
        if not Conv2dGw8.match(conv2d):
            raise ValueError(f"Conv2d {conv2d} does not match Conv2dGw8")
        module = Conv2dGw8(
            in_channels=conv2d.in_channels, out_channels=conv2d.out_channels,
            kernel_size=conv2d.kernel_size, stride=conv2d.stride, padding=conv2d.padding,
            groups=conv2d.groups, bias=conv2d.bias is not None, device=conv2d.weight.device,
        ).to(memory_format=torch.channels_last)  # fmt: skip
        module.weight = conv2d.weight
        module.bias = conv2d.bias
        return module

    def forward(self, x: torch.Tensor) -> torch.Tensor:  # pylint: disable=arguments-renamed
        padding_y, padding_x = _pair(self.padding)
        return conv2d_gw8(
            x, self.weight, self.bias, stride=1, padding_y=padding_y, padding_x=padding_x,
            groups=self.groups,
        )  # fmt: skip
