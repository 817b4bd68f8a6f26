"""`spio::layernorm_2d`: LayerNorm over the channels of an NCHW tensor with channels_last strides.

Forward runs the HIP kernel (csrc/layernorm_2d.hip; contract of the reference's
spio/src/layernorm_2d.cu:81-222).  The backward pass is written with torch operations in fp32 on
the same layout; it recomputes the statistics from the input.
"""

from typing import Optional, Tuple

import torch

from ..kernels.layernorm_2d_kernel import LayerNorm2dParams, layernorm_2d_kernel_factory


@torch.library.custom_op("spio::layernorm_2d", mutates_args=())
def layernorm_2d(inputs: torch.Tensor, weight: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, eps: float = 1e-6) -> torch.Tensor:  # fmt: skip
    """out[n,c,h,w] = (x - mean_c) * rsqrt(var_c + eps) * weight[c] + bias[c], fp16 in and out."""
    assert inputs.dim() == 4, "layernorm_2d takes an NCHW tensor"
    assert inputs.dtype == torch.float16, "layernorm_2d computes on float16 tensors"
    if inputs.device.type != "cuda":
        raise ValueError("spio::layernorm_2d runs on the GPU only")
    assert weight is None or (weight.dim() == 1 and weight.shape[0] == inputs.shape[1])
    assert bias is None or (bias.dim() == 1 and bias.shape[0] == inputs.shape[1])
    n, c, h, w = (int(v) for v in inputs.shape)
    params = LayerNorm2dParams(n=n, c=c, h=h, w=w, eps=float(eps),
                               has_weight=weight is not None, has_bias=bias is not None)  # fmt: skip
    x = inputs.contiguous(memory_format=torch.channels_last)
    out = torch.empty_like(x, memory_format=torch.channels_last)
    kernel = layernorm_2d_kernel_factory.get_kernel(params, inputs.device)
    kernel(out, x,
           None if weight is None else weight.detach().float().contiguous(),
           None if bias is None else bias.detach().float().contiguous())  # fmt: skip
    return out


@layernorm_2d.register_fake
def _layernorm_2d_fake(inputs, weight=None, bias=None, eps=1e-6):
    return torch.empty_like(inputs, memory_format=torch.channels_last)


def _setup_context(ctx, inputs, output):
    x, weight, bias, eps = inputs
    ctx.save_for_backward(x, weight)
    ctx.eps = eps
    ctx.has_bias = bias is not None


def _backward(ctx, grad_output) -> Tuple[Optional[torch.Tensor], ...]:
    x, weight = ctx.saved_tensors
    xf = x.float().permute(0, 2, 3, 1)  # [n, h, w, c] view of the channels_last tensor
    dy = grad_output.float().permute(0, 2, 3, 1)
    mean = xf.mean(-1, keepdim=True)
    var = (xf - mean).pow(2).mean(-1, keepdim=True)
    rstd = torch.rsqrt(var + ctx.eps)
    xhat = (xf - mean) * rstd
    g = dy if weight is None else dy * weight.float()
    dx = rstd * (g - g.mean(-1, keepdim=True) - xhat * (g * xhat).mean(-1, keepdim=True))
    grad_input = dx.permute(0, 3, 1, 2).to(x.dtype) if ctx.needs_input_grad[0] else None
    grad_weight = None
    if weight is not None and ctx.needs_input_grad[1]:
        grad_weight = (dy * xhat).sum((0, 1, 2)).to(weight.dtype)
    grad_bias = dy.sum((0, 1, 2)) if ctx.has_bias and ctx.needs_input_grad[2] else None
    return grad_input, grad_weight, grad_bias, None


layernorm_2d.register_autograd(_backward, setup_context=_setup_context)
