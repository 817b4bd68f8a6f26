"""GPU parity of the operator, its autograd, autocast, layer and registration.

Mirrors the function / layer / opcheck tests of the reference
(tests/test_conv2d_gw8.py:176-236; procedures spio/src_tests/run_test.py:128-246):
the op is called on fp32 arguments under torch.autocast so the AutocastCUDA
implementation runs, gradients come from torch.autograd.grad, and everything is
compared with the fp32 CPU oracle.
"""

import os

import pytest
import torch
from torch import nn

from helpers import random_params, sample_params, to_gpu
from oracle import conv2d_gw8_oracle as oracle
from spio_amd.functional import conv2d_gw8
from spio_amd.kernels import Conv2dGw8Params, Conv2dStats
from spio_amd.layers import Conv2dGw8

pytestmark = pytest.mark.gpu

FUNCTION_SHAPES = [
    Conv2dGw8Params(n=4, c=128, h=32, w=32, padding=(2, 0), r=4, s=1, has_bias=True),
    Conv2dGw8Params(n=4, c=64, h=16, w=32, padding=1, r=3, s=3, has_bias=True),
    Conv2dGw8Params(n=3, c=40, h=9, w=9, padding=2, r=5, s=5, has_bias=False),
    Conv2dGw8Params(n=1, c=128, h=64, w=64, padding=7, has_bias=False),
]


def _call(params, x, w, b):
    return conv2d_gw8(x, w, b, stride=1, padding_y=params.padding_h, padding_x=params.padding_w,
                      groups=params.groups)  # fmt: skip


def _depths(params):
    return Conv2dStats(params, output_names=["output", "grad_input", "grad_weight", "grad_bias"]).accumulation_depths


def run_function_test(params, seed=0):
    x, w, b, _dy = oracle.make_args(params.n, params.c, params.h, params.w, params.r, params.s,
                                    params.padding_h, params.padding_w, params.has_bias, seed)  # fmt: skip
    expected = oracle.fprop_torch(x, w, b, params.padding_h, params.padding_w)
    # fp32 arguments under autocast: exercises the AutocastCUDA implementation.
    xg, wg, bg = to_gpu(x).float(), to_gpu(w).float(), to_gpu(b)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = _call(params, xg, wg, bg)
    assert y.dtype == torch.float32  # cast back to the input dtype
    oracle.check_close(y, expected, acc_depth=_depths(params)[0], what=f"function {params.encode()}")
    # fp16 arguments without autocast
    y16 = _call(params, to_gpu(x), to_gpu(w), bg)
    assert y16.dtype == torch.float16 and y16.is_contiguous(memory_format=torch.channels_last)
    oracle.check_close(y16, expected, acc_depth=_depths(params)[0], what=f"function fp16 {params.encode()}")


def run_grad_function_test(params, seed=0):
    x, w, b, dy = oracle.make_args(params.n, params.c, params.h, params.w, params.r, params.s,
                                   params.padding_h, params.padding_w, params.has_bias, seed)  # fmt: skip
    dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, params.padding_h, params.padding_w)
    xg = to_gpu(x).float().requires_grad_(True)
    wg = to_gpu(w).float().requires_grad_(True)
    bg = to_gpu(b).requires_grad_(True) if b is not None else None
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = _call(params, xg, wg, bg)
    leaves = [xg, wg] + ([bg] if bg is not None else [])
    grads = torch.autograd.grad(y, leaves, to_gpu(dy).float())
    d = _depths(params)
    oracle.check_close(grads[0], dx_e, acc_depth=d[1], what=f"grad_input {params.encode()}")
    oracle.check_close(grads[1], dw_e, acc_depth=d[2], what=f"grad_weight {params.encode()}")
    assert grads[1].dtype == torch.float32
    if bg is not None:
        oracle.check_close(grads[2], db_e, acc_depth=d[3], what=f"grad_bias {params.encode()}")


@pytest.mark.parametrize("params", FUNCTION_SHAPES, ids=lambda p: p.encode())
def test_function(params):
    run_function_test(params)


@pytest.mark.parametrize("params", FUNCTION_SHAPES, ids=lambda p: p.encode())
def test_function_grad(params):
    run_grad_function_test(params)


@pytest.mark.slow
@pytest.mark.parametrize("params", sample_params(seed=4, count=6), ids=lambda p: p.encode())
def test_function_sampled(params):
    run_function_test(params, seed=1)
    run_grad_function_test(params, seed=1)


_RANDOM = random_params(int(os.environ.get("SPIO_RANDOM_SEED", "7")) + 100,
                        int(os.environ.get("SPIO_RANDOM_FUNCTION_SHAPES", "6")))  # fmt: skip


@pytest.mark.parametrize("params", _RANDOM, ids=lambda p: p.encode())
def test_function_random_shapes(params):
    """The operator and its autograd on seeded random shapes outside the reference's list (the
    kernels and tile configurations the operator itself selects, fused or separate backward)."""
    run_function_test(params, seed=2)
    run_grad_function_test(params, seed=2)


def test_backward_op_skips_what_is_not_needed():
    p = Conv2dGw8Params(n=2, c=16, h=8, w=8, has_bias=True)
    x, w, b, dy = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, True, 0)
    args = (to_gpu(x), to_gpu(w), to_gpu(b), to_gpu(dy), 1, 1)
    dx, dw, db = torch.ops.spio.conv2d_gw8_backward(*args, False, True, False)
    assert dx is None and db is None and dw.dtype == torch.float32 and dw.shape == w.shape
    _dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, 1, 1)
    # weight gradient without bias gradient: the fused kernel gets a null grad_bias pointer
    oracle.check_close(dw, dw_e, acc_depth=2 * 8 * 8, what="dw only")
    dx, dw, db = torch.ops.spio.conv2d_gw8_backward(*args, True, False, True)
    assert dw is None and dx.dtype == torch.float16 and db.dtype == torch.float32
    # bias gradient without weight gradient: the separate reduction
    oracle.check_close(db, db_e, acc_depth=2 * 8 * 8, what="db only")
    # both: grad_bias comes out of the weight-gradient kernel's own pass over grad_output
    dx, dw, db = torch.ops.spio.conv2d_gw8_backward(*args, False, True, True)
    assert dx is None
    oracle.check_close(dw, dw_e, acc_depth=2 * 8 * 8, what="dw fused")
    oracle.check_close(db, db_e, acc_depth=2 * 8 * 8, what="db fused")
    # only the input requires grad
    xg = to_gpu(x).requires_grad_(True)
    y = _call(p, xg, to_gpu(w), to_gpu(b))
    (gx,) = torch.autograd.grad(y, (xg,), to_gpu(dy))
    oracle.check_close(gx, oracle.grads_torch(x, w, b, dy, 1, 1)[0], acc_depth=72, what="dx only")


@pytest.mark.parametrize("mode", ["0", "1"])
def test_backward_op_fused_and_separate_kernels_agree_with_the_oracle(monkeypatch, mode):
    """SPIO_FUSED_BACKWARD=1 routes the backward op through the fused data+weight(+bias)
    gradient kernel, =0 through the separate kernels; both must match the oracle."""
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", mode)
    for p in (Conv2dGw8Params(n=3, c=40, h=12, w=20, padding=1, has_bias=True),
              Conv2dGw8Params(n=2, c=16, h=9, w=9, r=5, s=5, padding=2, has_bias=False),
              # output smaller and larger than the input
              Conv2dGw8Params(n=3, c=40, h=12, w=20, padding=0, has_bias=True),
              Conv2dGw8Params(n=2, c=16, h=9, w=9, r=5, s=3, padding=(3, 2), has_bias=True),
              # even filter sizes (the reference's regression shape, tests/test_conv2d_gw8.py:176-180)
              Conv2dGw8Params(n=4, c=128, h=32, w=32, r=4, s=1, padding=(2, 0), has_bias=True)):  # fmt: skip
        x, w, b, dy = oracle.make_args(p.n, p.c, p.h, p.w, p.r, p.s, p.padding_h, p.padding_w, p.has_bias, 3)
        dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, p.padding_h, p.padding_w)
        dx, dw, db = torch.ops.spio.conv2d_gw8_backward(
            to_gpu(x), to_gpu(w), to_gpu(b), to_gpu(dy), p.padding_h, p.padding_w, True, True, p.has_bias
        )
        depth = p.n * p.p * p.q
        oracle.check_close(dx, dx_e, acc_depth=8 * p.r * p.s, what=f"dx mode {mode}")
        oracle.check_close(dw, dw_e, acc_depth=depth, what=f"dw mode {mode}")
        if p.has_bias:
            oracle.check_close(db, db_e, acc_depth=depth, what=f"db mode {mode}")


def test_fused_backward_choice(monkeypatch):
    from spio_amd.functional import fused_backward_kernel

    dev = torch.device("cuda", 0)
    same = Conv2dGw8Params(n=2, c=16, h=8, w=8, padding=1)
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", "0")
    assert fused_backward_kernel(same, dev) is None
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", "1")
    assert fused_backward_kernel(same, dev) is not None
    assert fused_backward_kernel(Conv2dGw8Params(n=2, c=16, h=8, w=8, padding=0), dev) is not None
    assert fused_backward_kernel(Conv2dGw8Params(n=2, c=16, h=8, w=8, r=4, s=1, padding=(2, 0)), dev) is not None
    # 7x7 has no fused configuration: the separate kernels
    assert fused_backward_kernel(Conv2dGw8Params(n=2, c=16, h=8, w=8, r=7, s=7, padding=3), dev) is None
    # no recorded times for this shape and far fewer workgroups than compute units: separate kernels
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", "auto")
    assert fused_backward_kernel(same, dev) is None


def test_atomic_kernels_accumulate_and_two_stage_kernels_overwrite():
    """A weight-gradient (or fused backward) kernel that publishes with atomics adds to
    grad_weight: two launches give twice one launch's contribution (up to the order of fp32
    atomics).  A two-stage kernel stores grad_weight (and grad_bias) whole: whatever they held
    before is gone, which is why the operator does not zero them for such a kernel."""
    from spio_amd.hip import get_device_attributes
    from spio_amd.kernels import (
        Conv2dGw8BgradConfig,
        Conv2dGw8WgradConfig,
        conv2d_gw8_bgrad_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )

    attr = get_device_attributes(0)
    p = Conv2dGw8Params(n=6, c=16, h=8, w=8, has_bias=True)
    x, w, b, dy = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, True, 0)
    _dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, 1, 1)
    xg, wg, dyg = to_gpu(x), to_gpu(w), to_gpu(dy)

    def fresh(value):
        dw = torch.full(p.weight_shape, value, device="cuda").contiguous(memory_format=torch.channels_last)
        return dw, torch.full((p.c,), value, device="cuda")

    for two_stage in (0, 1):
        wk = conv2d_gw8_wgrad_kernel_factory.make_kernel(
            p, Conv2dGw8WgradConfig(groups=2, block_h=4, block_n=2, prefetch=2, two_stage=two_stage), attr)
        bk = conv2d_gw8_bgrad_kernel_factory.make_kernel(
            p, Conv2dGw8BgradConfig(groups=2, block_h=4, block_n=2, prefetch=2, two_stage=two_stage), attr)
        for kernel, call in ((wk, lambda dw, db: wk(dw, xg, dyg, db)),
                             (bk, lambda dw, db: bk(torch.empty_like(xg), dw, xg, dyg, wg, db))):  # fmt: skip
            kernel.compile()
            kernel.load(0)
            assert kernel.kernel_spec.overwrites_output == bool(two_stage)
            dw, db = fresh(0.0)
            call(dw, db)
            once_w, once_b = dw.clone(), db.clone()
            oracle.check_close(once_w, dw_e, acc_depth=p.n * 64, what=f"{kernel.kernel_name} once")
            oracle.check_close(once_b, db_e, acc_depth=p.n * 64, what=f"{kernel.kernel_name} bias once")
            call(dw, db)
            torch.cuda.synchronize()
            factor = 1 if two_stage else 2
            assert torch.allclose(dw, factor * once_w, rtol=1e-5, atol=1e-4)
            # grad_bias: the fused kernel's second stage stores it; the weight-gradient kernel's
            # two-stage mode still adds it with atomics
            bias_factor = 1 if (two_stage and kernel is bk) else 2
            assert torch.allclose(db, bias_factor * once_b, rtol=1e-5, atol=1e-3)
            if two_stage:  # garbage in the outputs does not matter
                dw, db = fresh(123.0)
                if kernel is wk:
                    db.zero_()
                call(dw, db)
                torch.cuda.synchronize()
                assert torch.allclose(dw, once_w, rtol=1e-5, atol=1e-4)
                assert torch.allclose(db, once_b, rtol=1e-5, atol=1e-3)
            kernel.unload()


def test_non_channels_last_arguments_are_accepted():
    """NCHW-contiguous inputs and weights are converted, like the reference's to_channels_last."""
    p = Conv2dGw8Params(n=2, c=16, h=8, w=8)
    x, w, _b, _dy = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, False, 0)
    y = _call(p, x.contiguous().cuda(), w.contiguous().cuda(), None)
    oracle.check_close(y, oracle.fprop_torch(x, w, None, 1, 1), acc_depth=72, what="nchw args")


@pytest.mark.parametrize("torchcompile", [False, True])
def test_layer(torchcompile):
    """An nn.Conv2d and the Conv2dGw8 sharing its parameters give the same result."""
    torch.manual_seed(0)
    conv = nn.Conv2d(64, 64, 3, padding=1, groups=8).cuda().to(memory_format=torch.channels_last)
    layer = Conv2dGw8.from_torch_module(conv)
    run = torch.compile(layer) if torchcompile else layer
    x = torch.randn(4, 64, 20, 24, device="cuda").contiguous(memory_format=torch.channels_last)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = run(x)
    expected = oracle.fprop_torch(x.half(), conv.weight.half(), conv.bias, 1, 1)
    oracle.check_close(y, expected, acc_depth=72, what="layer")


def test_layer_training_step():
    """fp32 master weights + autocast: gradients land in fp32 on the parameters."""
    torch.manual_seed(1)
    layer = Conv2dGw8(32, 32, 3, padding=1, groups=4).cuda().to(memory_format=torch.channels_last)
    x = torch.randn(2, 32, 12, 12, device="cuda").contiguous(memory_format=torch.channels_last)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = layer(x)
    dy = torch.randn_like(y)
    y.backward(dy)
    assert layer.weight.grad.dtype == torch.float32 and layer.bias.grad.dtype == torch.float32
    _dx, dw_e, db_e = oracle.grads_torch(x.half(), layer.weight.detach().half(), layer.bias.detach(), dy.half(), 1, 1)
    oracle.check_close(layer.weight.grad, dw_e, acc_depth=2 * 12 * 12, what="layer dw")
    oracle.check_close(layer.bias.grad, db_e, acc_depth=2 * 12 * 12, what="layer db")


@pytest.mark.parametrize("mode", ["0", "1"])
def test_two_layer_training_step(monkeypatch, mode):
    """Two stacked layers: the second one's backward needs grad_input, grad_weight and grad_bias,
    which is where the fused backward kernel runs (mode 1) or the separate kernels (mode 0).
    Gradients of both layers against the same network built from nn.Conv2d in fp32 on the CPU."""
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", mode)
    torch.manual_seed(2)
    c, groups = 48, 6
    net = nn.Sequential(Conv2dGw8(c, c, 3, padding=1, groups=groups), nn.ReLU(),
                        Conv2dGw8(c, c, 5, padding=2, groups=groups))  # fmt: skip
    ref = nn.Sequential(nn.Conv2d(c, c, 3, padding=1, groups=groups), nn.ReLU(),
                        nn.Conv2d(c, c, 5, padding=2, groups=groups))  # fmt: skip
    ref.load_state_dict({k: v.half().float() if v.dim() == 4 else v for k, v in net.state_dict().items()})
    net = net.cuda().to(memory_format=torch.channels_last)
    x = torch.randn(3, c, 14, 18).half()
    dy = torch.randn(3, c, 14, 18).half()
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = net(x.cuda().contiguous(memory_format=torch.channels_last))
    y.backward(dy.cuda())
    y_ref = ref(x.float())
    y_ref.backward(dy.float())
    # fp16 activations between the layers: compare with a tolerance scaled to the gradients' size
    for (name, p_gpu), (_n, p_ref) in zip(net.named_parameters(), ref.named_parameters()):
        got, want = p_gpu.grad.float().cpu(), p_ref.grad
        assert got.shape == want.shape
        err = (got - want).abs().max().item()
        assert err <= 2e-2 + 5e-3 * want.abs().max().item(), f"{name} mode {mode}: max err {err}"


@pytest.mark.parametrize("mode", ["0", "1"])
def test_ops_replay_correctly_from_a_hip_graph(monkeypatch, mode):
    """Forward and backward ops captured once into a HIP graph, replayed three times on new
    data with eager work and synchronisations between the replays; every replay must match the
    oracle (the launches go to the capturing stream and carry no memset nodes)."""
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", mode)
    p = Conv2dGw8Params(n=2, c=32, h=12, w=12, padding=1, has_bias=True)
    x0, w0, b0, dy0 = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, True, 0)
    x, w, b, dy = to_gpu(x0), to_gpu(w0), to_gpu(b0), to_gpu(dy0)

    def run():
        y = conv2d_gw8(x, w, b, 1, 1, 1, 1, p.groups)
        dx, dw, db = torch.ops.spio.conv2d_gw8_backward(x, w, b, dy, 1, 1, True, True, True)
        return y, dx, dw, db

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # first use outside the capture: kernel compilation and loading
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = run()
    torch.cuda.current_stream().wait_stream(side)
    for trial in range(3):
        xt, wt, bt, dyt = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, True, 10 + trial)
        x.copy_(to_gpu(xt)), w.copy_(to_gpu(wt)), b.copy_(to_gpu(bt)), dy.copy_(to_gpu(dyt))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        y_e = oracle.fprop_torch(xt, wt, bt, 1, 1)
        dx_e, dw_e, db_e = oracle.grads_torch(xt, wt, bt, dyt, 1, 1)
        what = f"graph replay {trial} mode {mode}"
        oracle.check_close(outs[0], y_e, acc_depth=72, what=what + " y")
        oracle.check_close(outs[1], dx_e, acc_depth=72, what=what + " dx")
        oracle.check_close(outs[2], dw_e, acc_depth=p.n * p.p * p.q, what=what + " dw")
        oracle.check_close(outs[3], db_e, acc_depth=p.n * p.p * p.q, what=what + " db")


def test_opcheck():
    p = Conv2dGw8Params(n=4, c=64, h=16, w=32, padding=1, has_bias=True)
    x, w, b, _ = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, True, 0)
    args = (to_gpu(x).requires_grad_(True), to_gpu(w).requires_grad_(True), to_gpu(b).requires_grad_(True))
    kwargs = dict(stride=1, padding_y=1, padding_x=1, dilation=1, groups=p.groups)
    torch.library.opcheck(conv2d_gw8, args, kwargs)


def test_compiled_training_step():
    """torch.compile of a layer, forward and backward: the fake implementations of both ops
    (shapes, strides, fp32 grad_weight) must agree with what the real ops return."""
    torch.manual_seed(2)
    layer = Conv2dGw8(32, 32, 3, padding=1, groups=4).cuda().to(memory_format=torch.channels_last)
    compiled = torch.compile(layer)
    x = torch.randn(2, 32, 10, 12, device="cuda").contiguous(memory_format=torch.channels_last).requires_grad_(True)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = compiled(x)
    dy = torch.randn_like(y)
    y.backward(dy)
    dx_e, dw_e, db_e = oracle.grads_torch(x.detach().half(), layer.weight.detach().half(), layer.bias.detach(),
                                          dy.half(), 1, 1)  # fmt: skip
    oracle.check_close(x.grad, dx_e, acc_depth=72, what="compiled dx")
    oracle.check_close(layer.weight.grad, dw_e, acc_depth=2 * 10 * 12, what="compiled dw")
    oracle.check_close(layer.bias.grad, db_e, acc_depth=2 * 10 * 12, what="compiled db")


def test_kernel_launch_argument_errors():
    """Launch-time checks raise ValueError, as the reference's Kernel.launch does
    (spio/kernels/kernel.py:135-151): tensors that are not channels_last, CPU tensors."""
    from spio_amd.kernels import conv2d_gw8_kernel_factory

    p = Conv2dGw8Params(n=2, c=16, h=8, w=8)
    x, w, _b, _dy = oracle.make_args(p.n, p.c, p.h, p.w, 3, 3, 1, 1, False, 0)
    kernel = conv2d_gw8_kernel_factory.get_kernel(p, torch.device("cuda", 0))
    out = torch.empty(p.output_shape, device="cuda", dtype=torch.float16).contiguous(memory_format=torch.channels_last)
    with pytest.raises(ValueError, match="Error in kernel"):
        kernel(out, x.contiguous().cuda(), to_gpu(w), None)  # NCHW-contiguous input
    with pytest.raises(ValueError, match="Error in kernel"):
        kernel(out, x, to_gpu(w), None)  # CPU tensor among GPU tensors
    kernel(out, to_gpu(x), to_gpu(w), None)  # and the right call still works
    oracle.check_close(out, oracle.fprop_torch(x, w, None, 1, 1), acc_depth=72, what="after errors")
