"""MI355X-native implementation of Spio's grouped-width-8 conv2d path.

Public surface (same names as the reference package `spio`):
  spio_amd.functional.conv2d_gw8         custom op with autograd / autocast / fake impls
  spio_amd.layers.Conv2dGw8, make_conv2d nn.Conv2d drop-in layer
  spio_amd.transform.transform           replaces matching nn.Conv2d modules in a model
  spio_amd.kernels                       params, stats, kernel factories, tuner
"""

__version__ = "0.1.0"

supported_arch = ("gfx950",)
