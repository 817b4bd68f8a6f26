"""`spio::layernorm_2d`: LayerNorm over the channels of an NCHW tensor with channels_last strides.

Forward runs the HIP kernel (csrc/layernorm_2d.hip; contract of the reference's
spio/src/layernorm_2d.cu:81-222).  The backward pass runs a second HIP kernel
(csrc/layernorm_2d_bwd.hip: grad_input and per-workgroup partial sums of grad_weight and
grad_bias in one pass over the input and grad_output, statistics recomputed from the input, and a
small second stage that adds the partial sums).  Shapes that kernel does not take (more than
1024 channels) and SPIO_LAYERNORM_BACKWARD=torch use torch operations in fp32 on the same layout.
"""

from typing import Optional, Tuple

import torch

import os

from ..kernels.layernorm_2d_kernel import (
    LayerNorm2dParams,
    layernorm_2d_bwd_is_supported,
    layernorm_2d_bwd_kernel_factory,
    layernorm_2d_kernel_factory,
)


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


@torch.library.custom_op("spio::layernorm_2d_backward", mutates_args=())
def layernorm_2d_backward(inputs: torch.Tensor, grad_output: torch.Tensor, weight: Optional[torch.Tensor],
                          eps: float) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    """(grad_input fp16, [grad_weight; grad_bias] fp32 as one [2, C] tensor) of layernorm_2d: the
    backward kernel and its small second stage that adds the workgroups' partial rows."""
    n, c, h, w = (int(v) for v in inputs.shape)
    params = LayerNorm2dParams(n=n, c=c, h=h, w=w, eps=float(eps), has_weight=weight is not None, has_bias=False)
    x = inputs.contiguous(memory_format=torch.channels_last)
    dy = grad_output.to(torch.float16).contiguous(memory_format=torch.channels_last)
    kernel = layernorm_2d_bwd_kernel_factory.get_kernel(params, inputs.device)
    grad_input = torch.empty_like(x, memory_format=torch.channels_last)
    sums = torch.empty((2, c), dtype=torch.float32, device=inputs.device)
    kernel(sums, grad_input, x, dy, None if weight is None else weight.detach().float().contiguous())
    return grad_input, sums


@layernorm_2d_backward.register_fake
def _layernorm_2d_backward_fake(inputs, grad_output, weight, eps):
    c = inputs.shape[1]
    return (torch.empty_like(inputs, memory_format=torch.channels_last),
            inputs.new_empty((2, c), dtype=torch.float32))  # fmt: skip


def _backward(ctx, grad_output) -> Tuple[Optional[torch.Tensor], ...]:
    x, weight = ctx.saved_tensors
    n, c, h, w = (int(v) for v in x.shape)
    use_kernel = (os.environ.get("SPIO_LAYERNORM_BACKWARD", "hip") != "torch" and x.device.type == "cuda"
                  and layernorm_2d_bwd_is_supported(LayerNorm2dParams(n=n, c=c, h=h, w=w)))  # fmt: skip
    if use_kernel:
        grad_input, sums = layernorm_2d_backward(x, grad_output, weight, ctx.eps)
        return (
            grad_input if ctx.needs_input_grad[0] else None,
            sums[0].to(weight.dtype) if weight is not None and ctx.needs_input_grad[1] else None,
            sums[1] if ctx.has_bias and ctx.needs_input_grad[2] else None,
            None,
        )
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
