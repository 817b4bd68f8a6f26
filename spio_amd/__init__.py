"""MI355X-native implementation of Spio's grouped-width-8 conv2d path.

Public surface (same names as the reference package `spio`):
  spio_amd.functional.conv2d_gw8         custom op with autograd / autocast / fake impls
  spio_amd.layers.Conv2dGw8, make_conv2d nn.Conv2d drop-in layer
  spio_amd.transform.transform           replaces matching nn.Conv2d modules in a model
  spio_amd.kernels                       params, stats, kernel factories, tuner
"""

__version__ = "0.1.0"

supported_arch = ("gfx950",)


def install_as_spio():
    """Make `import spio...` resolve to this package (for code written against the reference).

    Registers `spio` and its sub-packages `functional`, `layers`, `kernels`, `transform`,
    `util`, `compiler` as aliases of the spio_amd modules.  Refuses to shadow a real `spio`.
    """
    import importlib
    import sys

    existing = sys.modules.get("spio")
    if existing is not None and not getattr(existing, "__file__", "").startswith(__path__[0]):
        raise RuntimeError("a different 'spio' package is already imported")
    this = sys.modules[__name__]
    sys.modules["spio"] = this
    for name in ("functional", "layers", "kernels", "transform", "util", "compiler"):
        module = importlib.import_module(f"{__name__}.{name}")
        sys.modules[f"spio.{name}"] = module
        setattr(this, name, module)
    return this
