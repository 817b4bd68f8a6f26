"""`spio::conv2d_gw8` and `spio::conv2d_gw8_backward` custom operators.

Same operator names, schemas, dtype rules and autograd wiring as the
reference (spio/functional/conv2d_gw8_function.py:17-233):
  * inputs and weight fp16, bias fp32 or None, unit stride and dilation,
    groups == C // 8; violations raise AssertionError (:46-51);
  * the output is a fresh fp16 channels_last tensor (:53-58);
  * backward returns (grad_input fp16, grad_weight fp32, grad_bias fp32), each
    None when not needed (:124-147);
  * under torch.autocast("cuda") arguments of any float dtype are cast to
    fp16 (bias to fp32) and the result is cast back (:67-80, 232-233).
One deliberate difference: the fake implementation of the backward op reports
grad_weight as fp32, which is what the real op returns (the reference's fake
says fp16, :164).

When grad_input and grad_weight are both wanted, the backward op can run one
fused kernel that reads grad_output once instead of the reference's two
launches (:119-146).  SPIO_FUSED_BACKWARD=0 never fuses, =1 fuses whenever the
shape has a fused configuration, anything else (default) fuses
when the recorded kernel times say it is faster, or, without records, when the
fused kernel has enough workgroups to fill the device.
"""

import os
import threading

from typing import Tuple

import torch

from ..hip import get_device_attributes
from ..kernels import (
    Conv2dGw8Params,
    bgrad_is_supported,
    conv2d_gw8_bgrad_kernel_factory,
    conv2d_gw8_kernel_factory,
    conv2d_gw8_wgrad_kernel_factory,
    tuner,
)
from ..util import to_channels_last

_fused_choice = {}
LAUNCH_GAP_US = 2.2  # an empty kernel in a back-to-back launch loop on MI355X
_fused_choice_lock = threading.Lock()


def fused_backward_kernel(params: Conv2dGw8Params, device):
    """The fused data+weight gradient kernel if it should run for `params`, else None."""
    mode = os.environ.get("SPIO_FUSED_BACKWARD", "auto").strip().lower()
    if mode in ("0", "false", "off", "no") or not bgrad_is_supported(params):
        return None
    ordinal = device.index if device.index is not None else torch.cuda.current_device()
    key = (params, ordinal, mode)
    with _fused_choice_lock:
        if key in _fused_choice:
            return _fused_choice[key]
    attr = get_device_attributes(ordinal)
    fused = None
    if list(conv2d_gw8_bgrad_kernel_factory.configs(params, attr)):
        fused = conv2d_gw8_bgrad_kernel_factory.get_kernel(params, device)
        if mode not in ("1", "true", "on", "yes"):
            # the separate kernels, tuned or looked up the same way, for the comparison
            conv2d_gw8_kernel_factory.get_kernel(params, device, igrad=True)
            conv2d_gw8_wgrad_kernel_factory.get_kernel(params, device)
            times = [
                (tuner.lookup(attr, f.get_full_kernel_name(params, **kw)) or {}).get("us")
                for f, kw in ((conv2d_gw8_bgrad_kernel_factory, {}),
                              (conv2d_gw8_kernel_factory, {"igrad": True}),
                              (conv2d_gw8_wgrad_kernel_factory, {}))
            ]  # fmt: skip
            if all(t is not None for t in times):
                # one launch instead of two: the second launch costs about what an empty kernel
                # does in a back-to-back stream (measured at N=32, C=64, 56x56: the step with the
                # fused kernel takes 25.6 us, with the two separate ones, whose times add up to
                # 0.5 us less, 30.3 us)
                if times[0] >= times[1] + times[2] + LAUNCH_GAP_US:
                    fused = None
            elif fused.kernel_spec.launch_params.grid[0] < 0.75 * attr.multiprocessor_count:
                fused = None  # no measurements: too few workgroups to fill the device
    with _fused_choice_lock:
        _fused_choice[key] = fused
    return fused


def reset_fused_backward_choices():
    """Forget which shapes run the fused backward kernel (after the tuning records changed)."""
    with _fused_choice_lock:
        _fused_choice.clear()


def _is_unit(value) -> bool:
    return value in (1, (1, 1))


def _require_gpu(tensor: torch.Tensor):
    if tensor.device.type != "cuda":
        raise RuntimeError(
            "spio::conv2d_gw8 runs on the GPU only: its HIP kernels have no CPU fallback "
            f"(got a tensor on {tensor.device})"
        )


@torch.library.custom_op("spio::conv2d_gw8", mutates_args=())
def conv2d_gw8(
    inputs: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor = None,
    stride: int = 1,
    padding_y: int = 0,
    padding_x: int = 0,
    dilation: int = 1,
    groups: int = 1,
) -> torch.Tensor:
    """conv2d with group width 8, channels_last fp16.

    Args:
        inputs: (N, C, H, W) fp16.
        weight: (C, 8, R, S) fp16.
        bias: optional (C,) fp32.
        stride, dilation: must be 1.
        padding_y, padding_x: zero padding of height and width.
        groups: must equal C // 8.

    Returns:
        (N, C, P, Q) fp16, channels_last.
    """
    assert inputs.dtype == torch.float16
    assert weight.dtype == torch.float16
    assert bias is None or bias.dtype == torch.float32
    assert _is_unit(stride)
    assert _is_unit(dilation)
    assert groups == inputs.shape[1] // 8
    _require_gpu(inputs)
    params = Conv2dGw8Params.from_tensors(inputs, weight, bias, (padding_y, padding_x))
    output = torch.empty(
        params.output_shape, device=inputs.device, dtype=torch.float16,
        memory_format=torch.channels_last,
    )  # fmt: skip
    inputs, weight = to_channels_last(inputs, weight)
    if bias is not None:
        bias = bias.contiguous()
    kernel = conv2d_gw8_kernel_factory.get_kernel(params, inputs.device)
    kernel(output, inputs, weight, bias)
    return output


# Autocast support for custom ops: https://github.com/pytorch/pytorch/issues/137033
def conv2d_gw8_autocast(ks, inputs, weight, bias, *args, **kwargs):
    """AutocastCUDA implementation: cast, redispatch below autocast, cast back."""
    input_dtype = inputs.dtype
    inputs = inputs.to(dtype=torch.float16)
    weight = weight.to(dtype=torch.float16)
    if bias is not None:
        bias = bias.to(dtype=torch.float32)
    autocast = torch._C.DispatchKeySet("AutocastCUDA")
    with torch._C._ExcludeDispatchKeyGuard(autocast):
        result = torch.ops.spio.conv2d_gw8.default.redispatch(
            ks - autocast, inputs, weight, bias, *args, **kwargs
        )
    return result.to(dtype=input_dtype)


@conv2d_gw8.register_fake
def _conv2d_gw8_fake(
    inputs, weight, bias=None, stride: int = 1, padding_y: int = 0, padding_x: int = 0,
    dilation: int = 1, groups: int = 1,
):  # fmt: skip
    assert _is_unit(stride)
    assert _is_unit(dilation)
    assert groups == inputs.shape[1] // 8
    params = Conv2dGw8Params.from_tensors(inputs, weight, bias, (padding_y, padding_x))
    return inputs.new_empty(params.output_shape).to(memory_format=torch.channels_last)


@torch.library.custom_op("spio::conv2d_gw8_backward", mutates_args=())
def conv2d_gw8_backward_op(
    inputs: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    grad_output: torch.Tensor,
    padding_y: int,
    padding_x: int,
    needs_input_grad: bool,
    needs_weight_grad: bool,
    needs_bias_grad: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gradients of conv2d_gw8 with respect to inputs, weight and bias."""
    assert grad_output.dtype == torch.float16
    assert inputs.dtype == torch.float16
    assert weight.dtype == torch.float16
    _require_gpu(inputs)

    grad_output, inputs, weight = to_channels_last(grad_output, inputs, weight)
    params = Conv2dGw8Params.from_tensors(inputs, weight, bias, padding=(padding_y, padding_x))
    assert tuple(grad_output.shape) == params.output_shape

    grad_bias = None
    grad_input = None
    fused = fused_backward_kernel(params, inputs.device) if needs_input_grad and needs_weight_grad else None
    if fused is not None:
        # one pass over grad_output for both gradients (and grad_bias when the layer has a bias);
        # atomic kernels add into zeroed tensors, two-stage ones store them whole
        make = torch.empty_like if fused.kernel_spec.overwrites_output else torch.zeros_like
        grad_weight = make(weight, dtype=torch.float32)
        grad_input = torch.empty_like(inputs)
        if params.has_bias:
            if needs_bias_grad:
                alloc = torch.empty if fused.kernel_spec.overwrites_output else torch.zeros
                grad_bias = alloc(params.c, dtype=torch.float32, device=inputs.device)
            fused(grad_input, grad_weight, inputs, grad_output, weight, grad_bias)
        else:
            fused(grad_input, grad_weight, inputs, grad_output, weight)
    elif needs_weight_grad:
        # An atomic kernel accumulates into grad_weight, so it starts from zero; a two-stage one
        # stores it whole; fp32.
        kernel = conv2d_gw8_wgrad_kernel_factory.get_kernel(params, inputs.device)
        make = torch.empty_like if kernel.kernel_spec.overwrites_output else torch.zeros_like
        grad_weight = make(weight, dtype=torch.float32)
        if params.has_bias:
            # With a bias the weight-gradient kernel also sums grad_output per channel while it
            # streams it (the reference runs a separate reduction, conv2d_gw8_function.py:134-136).
            if needs_bias_grad:
                grad_bias = torch.zeros(params.c, dtype=torch.float32, device=inputs.device)
            kernel(grad_weight, inputs, grad_output, grad_bias)
        else:
            kernel(grad_weight, inputs, grad_output)
    else:
        grad_weight = None

    if needs_bias_grad and grad_bias is None:
        grad_bias = grad_output.sum(dim=(0, 2, 3), dtype=torch.float32)

    if needs_input_grad and grad_input is None:
        grad_input = torch.empty_like(inputs)
        kernel = conv2d_gw8_kernel_factory.get_kernel(params, inputs.device, igrad=True)
        kernel(grad_input, grad_output, weight, None)
    return grad_input, grad_weight, grad_bias


@conv2d_gw8_backward_op.register_fake
def _conv2d_gw8_backward_fake(
    inputs, weight, bias, _grad_output, _padding_y, _padding_x,
    needs_input_grad, needs_weight_grad, needs_bias_grad,
):  # fmt: skip
    grad_weight = grad_bias = grad_input = None
    if needs_weight_grad:
        grad_weight = weight.new_empty(weight.shape, dtype=torch.float32).to(
            memory_format=torch.channels_last
        )
    if needs_bias_grad:
        grad_bias = bias.new_empty(bias.shape, dtype=torch.float32)
    if needs_input_grad:
        grad_input = inputs.new_empty(inputs.shape).to(memory_format=torch.channels_last)
    return grad_input, grad_weight, grad_bias


def conv2d_gw8_backward(ctx, grad_output):
    """Autograd backward: one call of the backward op for whatever is needed."""
    inputs, weight, bias = ctx.saved_tensors
    grad_input, grad_weight, grad_bias = conv2d_gw8_backward_op(
        inputs, weight, bias, grad_output, ctx.padding_y, ctx.padding_x,
        ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2],
    )  # fmt: skip
    return grad_input, grad_weight, grad_bias, None, None, None, None, None


def conv2d_gw8_setup_context(ctx, inputs, output):
    """Save what backward needs."""
    input_tensor, weight, bias, _stride, padding_y, padding_x, *_ = inputs
    assert input_tensor.dtype == torch.float16
    assert weight.dtype == torch.float16
    assert output.dtype == torch.float16
    if bias is not None:
        assert bias.dtype == torch.float32
    ctx.save_for_backward(input_tensor, weight, bias)
    ctx.padding_y = padding_y
    ctx.padding_x = padding_x


conv2d_gw8.register_autograd(conv2d_gw8_backward, setup_context=conv2d_gw8_setup_context)

_lib = torch.library.Library("spio", "FRAGMENT")
_lib.impl("conv2d_gw8", conv2d_gw8_autocast, "AutocastCUDA", with_keyset=True)
