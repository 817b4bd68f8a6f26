"""Parameters of one grouped-width-8 convolution.

Restates spio/kernels/conv2d_gw8_params.py:10-209: same fields, defaults,
`encode` format, derived shapes and transposed padding.  One deliberate
extension: kernel sizes up to 7 are accepted (the reference asserts 1..5,
conv2d_gw8_params.py:137-138) because the kernels here support them; the
layer-matching rule of `Conv2dGw8.match_args` keeps the reference's 1..5.
"""

import re
from dataclasses import dataclass
from typing import Tuple, Union

MAX_KERNEL_SIZE = 7


@dataclass(frozen=True)
class Conv2dGw8Params:
    """Shape of a conv2d with C_in == C_out == c, groups == c // 8, unit stride/dilation."""

    n: int
    c: int
    h: int
    w: int
    padding: Union[int, Tuple[int, int]] = 1
    r: int = 3
    s: int = 3
    has_bias: bool = False
    group_width: int = 8
    stride: int = 1

    def encode(self) -> str:
        """E.g. '32n_64c_56h_56w_1py_1px_3r_3s_nb' (conv2d_gw8_params.py:38-44)."""
        return (
            f"{self.n}n_{self.c}c_{self.h}h_{self.w}w_{self.padding_h}py_{self.padding_w}px_"
            f"{self.r}r_{self.s}s_{'b' if self.has_bias else 'nb'}"
        )

    _PATTERN = re.compile(r"(\d+)n_(\d+)c_(\d+)h_(\d+)w_(\d+)py_(\d+)px_(\d+)r_(\d+)s_(b|nb)$")

    @classmethod
    def decode(cls, string: str) -> "Conv2dGw8Params":
        """Inverse of encode(); raises ValueError on anything else."""
        m = cls._PATTERN.match(string)
        if m is None:
            raise ValueError("Invalid string representation.")
        n, c, h, w, py, px, r, s = (int(v) for v in m.groups()[:8])
        return cls(n=n, c=c, h=h, w=w, padding=(py, px), r=r, s=s, has_bias=m.group(9) == "b")

    @staticmethod
    def from_tensors(inputs, weight, bias, padding=1) -> "Conv2dGw8Params":
        """Derive and validate parameters from conv2d arguments."""
        assert bias is None or (bias.dim() == 1 and bias.shape[0] == weight.shape[0])
        n, c, h, w = inputs.shape
        k, group_width, r, s = weight.shape
        assert group_width == Conv2dGw8Params.group_width, "Only group width of 8 is supported."
        assert k == c, "Number of output channels must match number of input channels."
        params = Conv2dGw8Params(
            n=int(n), c=int(c), h=int(h), w=int(w), r=int(r), s=int(s),
            padding=padding, has_bias=bias is not None,
        )  # fmt: skip
        params.validate()
        return params

    @staticmethod
    def from_torch_module(module, inputs) -> "Conv2dGw8Params":
        """Parameters of an nn.Conv2d applied to `inputs` (not validated)."""
        n, c, h, w = inputs.shape
        k, _gw, r, s = module.weight.shape
        assert k == c, f"Number of output channels must match number of input channels. {k} != {c}"
        return Conv2dGw8Params(
            n=int(n), c=int(c), h=int(h), w=int(w), r=int(r), s=int(s),
            padding=module.padding, has_bias=module.bias is not None,
        )  # fmt: skip

    def is_valid(self) -> bool:
        """validate() as a predicate."""
        try:
            self.validate()
            return True
        except AssertionError:
            return False

    def validate(self):
        """Assert that the kernels support these parameters."""
        assert self.n > 0 and self.c > 0 and self.h > 0 and self.w > 0
        assert self.padding_h >= 0 and self.padding_w >= 0
        assert self.c % self.group_width == 0, "Number of channels must be divisible by group width."
        assert self.group_width == 8 and self.stride == 1
        assert 1 <= self.r <= MAX_KERNEL_SIZE, f"Kernel height must be between 1 and {MAX_KERNEL_SIZE}."
        assert 1 <= self.s <= MAX_KERNEL_SIZE, f"Kernel width must be between 1 and {MAX_KERNEL_SIZE}."
        assert self.p > 0 and self.q > 0, "Output would be empty."

    @property
    def groups(self) -> int:
        return self.c // self.group_width

    @property
    def padding_h(self) -> int:
        return self.padding[0] if isinstance(self.padding, tuple) else self.padding

    @property
    def padding_w(self) -> int:
        return self.padding[1] if isinstance(self.padding, tuple) else self.padding

    @property
    def transpose_padding_h(self) -> int:
        """Padding of the data-gradient convolution; negative when padding_h > r - 1."""
        return self.r - 1 - self.padding_h

    @property
    def transpose_padding_w(self) -> int:
        return self.s - 1 - self.padding_w

    @property
    def k(self) -> int:
        return self.c

    @property
    def p(self) -> int:
        return self.h + 2 * self.padding_h - self.r + 1

    @property
    def q(self) -> int:
        return self.w + 2 * self.padding_w - self.s + 1

    @property
    def kernel_size(self) -> Tuple[int, int]:
        return (self.r, self.s)

    @property
    def input_shape(self) -> Tuple[int, int, int, int]:
        return (self.n, self.c, self.h, self.w)

    @property
    def output_shape(self) -> Tuple[int, int, int, int]:
        return (self.n, self.k, self.p, self.q)

    @property
    def weight_shape(self) -> Tuple[int, int, int, int]:
        return (self.k, self.group_width, self.r, self.s)

    @property
    def bias_shape(self) -> Tuple[int]:
        return (self.k,)
