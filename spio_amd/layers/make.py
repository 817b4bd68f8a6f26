"""Layer construction by nn.Conv2d arguments (reference: spio/layers/make.py:6)."""

from .conv2d_gw8 import Conv2dGw8


def make_conv2d(*args, **kwargs):
    """A Conv2dGw8 for nn.Conv2d-style arguments, or None when they do not qualify."""
    return Conv2dGw8.make(*args, **kwargs)
