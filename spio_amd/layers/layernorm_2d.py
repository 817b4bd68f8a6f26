"""LayerNorm over the channel dimension of an NCHW tensor, as ConvNeXt-style blocks use it."""

import torch
from torch import nn
import torch.nn.functional as F

from ..functional.layernorm_2d_function import layernorm_2d


class LayerNorm2d(nn.LayerNorm):
    """`nn.LayerNorm(C)` applied to the channels of [N, C, H, W].

    float16 GPU tensors whose channel count is a multiple of 8 go through the
    `spio::layernorm_2d` kernel (NHWC in memory, one pass); everything else takes torch's
    layer_norm on the permuted tensor, which is the same function.
    """

    def forward(self, x: torch.Tensor) -> torch.Tensor:  # pylint: disable=arguments-renamed
        dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else x.dtype
        if (x.is_cuda and x.dim() == 4 and dtype == torch.float16 and x.shape[1] % 8 == 0
                and len(self.normalized_shape) == 1 and x.shape[1] <= 2048):  # fmt: skip
            return layernorm_2d(x.to(torch.float16), self.weight, self.bias, self.eps).to(x.dtype)
        y = F.layer_norm(x.permute(0, 2, 3, 1), self.normalized_shape, self.weight, self.bias, self.eps)
        return y.permute(0, 3, 1, 2)
