"""LayerNorm2d kernel (`spio::layernorm_2d`) against torch's layer_norm in fp32 on the CPU.

Contract of the reference's device source spio/src/layernorm_2d.cu:81-222 (NHWC fp16, fp32
statistics over C per pixel); the reference has no test for it, so torch is the oracle.
Tolerance: one fp16 rounding of an O(1..10) value plus fp32 statistics: rtol 2e-3, atol 4e-3.
"""

import os

import pytest
import torch
import torch.nn.functional as F

from spio_amd.functional import layernorm_2d
from spio_amd.hip import get_device_attributes
from spio_amd.kernels import (
    LayerNorm2dParams,
    layernorm_2d_bwd_is_supported,
    layernorm_2d_bwd_kernel_factory,
    layernorm_2d_kernel_factory,
)
from spio_amd.layers import LayerNorm2d

pytestmark = pytest.mark.gpu

SHAPES = [
    # the four widths of the network benchmark (small batch), then shapes that exercise lanes
    # without a unit (c/8 not a power of two), two units per lane, and a ragged last pass
    (4, 96, 56, 56), (4, 192, 28, 28), (8, 384, 14, 14), (16, 768, 7, 7),
    (3, 8, 5, 7), (2, 40, 9, 9), (1, 1000, 3, 5), (5, 64, 1, 1), (2, 2048, 2, 3),
]  # fmt: skip


def _reference(x, w, b, eps):
    y = F.layer_norm(x.float().permute(0, 2, 3, 1), (x.shape[1],), w, b, eps)
    return y.permute(0, 3, 1, 2)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("affine", ["wb", "w", "none"])
def test_layernorm_2d_matches_torch(shape, affine):
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(shape, generator=g) * 2 + 0.5).half()
    c = shape[1]
    w = torch.randn(c, generator=g) if affine != "none" else None
    b = torch.randn(c, generator=g) if affine == "wb" else None
    expected = _reference(x, w, b, 1e-6)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    out = layernorm_2d(xg, None if w is None else w.cuda(), None if b is None else b.cuda(), 1e-6)
    assert out.dtype == torch.float16 and out.is_contiguous(memory_format=torch.channels_last)
    torch.testing.assert_close(out.float().cpu(), expected, rtol=2e-3, atol=4e-3)


def test_every_configuration_of_one_shape():
    attr = get_device_attributes(0)
    params = LayerNorm2dParams(n=3, c=192, h=13, w=11)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(params.shape, generator=g).half()
    w, b = torch.randn(192, generator=g), torch.randn(192, generator=g)
    expected = _reference(x, w, b, params.eps)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    for config in layernorm_2d_kernel_factory.configs(params, attr):
        kernel = layernorm_2d_kernel_factory.make_kernel(params, config, attr)
        kernel.compile()
        kernel.load(0)
        out = torch.full_like(xg, -42.0)
        kernel(out, xg, w.cuda(), b.cuda())
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float().cpu(), expected, rtol=2e-3, atol=4e-3, msg=str(config))
        kernel.unload()


def _reference_backward(x, dy, w, b, eps):
    xr = x.float().requires_grad_(True)
    wr = None if w is None else w.clone().requires_grad_(True)
    br = None if b is None else b.clone().requires_grad_(True)
    _reference(xr, wr, br, eps).backward(dy.float())
    return xr.grad, None if wr is None else wr.grad, None if br is None else br.grad


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("affine", ["wb", "w", "none"])
def test_layernorm_2d_backward_matches_torch(shape, affine):
    """grad_input, grad_weight and grad_bias through the op's autograd (the backward kernel up to
    1024 channels, torch operations beyond) against torch's autograd in fp32 on the CPU.
    Tolerances: grad_input is one fp16 rounding of an O(1..10) value; the channel sums add up to
    12544 products in fp32 in another order."""
    g = torch.Generator().manual_seed(sum(shape) + 7)
    x = (torch.randn(shape, generator=g) * 2 + 0.5).half()
    dy = torch.randn(shape, generator=g).half()
    c = shape[1]
    w = torch.randn(c, generator=g) if affine != "none" else None
    b = torch.randn(c, generator=g) if affine == "wb" else None
    ex_dx, ex_dw, ex_db = _reference_backward(x, dy, w, b, 1e-6)
    xg = x.cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    wg = None if w is None else w.cuda().requires_grad_(True)
    bg = None if b is None else b.cuda().requires_grad_(True)
    out = layernorm_2d(xg, wg, bg, 1e-6)
    out.backward(dy.cuda().contiguous(memory_format=torch.channels_last))
    assert xg.grad.dtype == torch.float16
    torch.testing.assert_close(xg.grad.float().cpu(), ex_dx, rtol=4e-3, atol=4e-3)
    if w is not None:
        torch.testing.assert_close(wg.grad.cpu(), ex_dw, rtol=2e-3, atol=3e-2)
    if b is not None:
        torch.testing.assert_close(bg.grad.cpu(), ex_db, rtol=2e-3, atol=3e-2)


def test_every_backward_configuration_of_one_shape():
    attr = get_device_attributes(0)
    params = LayerNorm2dParams(n=3, c=192, h=13, w=11, has_bias=False)
    assert layernorm_2d_bwd_is_supported(params)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(params.shape, generator=g).half()
    dy = torch.randn(params.shape, generator=g).half()
    w = torch.randn(192, generator=g)
    ex_dx, ex_dw, ex_db = _reference_backward(x, dy, w, torch.zeros(192), params.eps)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    dyg = dy.cuda().contiguous(memory_format=torch.channels_last)
    configs = layernorm_2d_bwd_kernel_factory.configs(params, attr)
    assert {c.lanes for c in configs} == {0, 8}
    for config in configs:
        kernel = layernorm_2d_bwd_kernel_factory.make_kernel(params, config, attr)
        kernel.compile()
        kernel.load(0)
        dx = torch.full_like(xg, -42.0)
        sums = torch.full((2, 192), float("nan"), device="cuda")
        kernel(sums, dx, xg, dyg, w.cuda())
        torch.cuda.synchronize()
        torch.testing.assert_close(dx.float().cpu(), ex_dx, rtol=4e-3, atol=4e-3, msg=str(config))
        sums = sums.cpu()
        torch.testing.assert_close(sums[0], ex_dw, rtol=2e-3, atol=3e-2, msg=str(config))
        torch.testing.assert_close(sums[1], ex_db, rtol=2e-3, atol=3e-2, msg=str(config))
        kernel.unload()


def _random_layernorm_params(seed, count):
    import random

    rng = random.Random(seed)
    out = []
    while len(out) < count:
        c = 8 * rng.choice([1, 2, 3, 5, 8, 12, 24, 48, 96, 128, rng.randint(1, 128)])
        n, h, w = rng.randint(1, 9), rng.choice([1, 7, 14, rng.randint(1, 40)]), rng.choice([1, 7, 14, rng.randint(1, 40)])
        if n * c * h * w <= 2_000_000:
            out.append(LayerNorm2dParams(n=n, c=c, h=h, w=w, has_weight=rng.random() < 0.7, has_bias=rng.random() < 0.5,
                                         eps=rng.choice([1e-6, 1e-5, 1e-3])))  # fmt: skip
    return out


_RANDOM_LN = _random_layernorm_params(int(os.environ.get("SPIO_RANDOM_SEED", "7")),
                                      int(os.environ.get("SPIO_RANDOM_LAYERNORMS", "6")))  # fmt: skip


@pytest.mark.parametrize("params", _RANDOM_LN, ids=lambda p: p.encode())
def test_random_shapes_every_configuration_forward_and_backward(params):
    """Seeded random shapes (channel counts 8..1024 that are not powers of two, pixel counts that
    leave ragged passes, with and without weight and bias, three eps values): every legal
    configuration of the forward kernel and, where the shape has one, of the backward kernel."""
    attr = get_device_attributes(0)
    g = torch.Generator().manual_seed(params.n + params.c + params.h + params.w)
    x = (torch.randn(params.shape, generator=g) * 2 + 0.5).half()
    dy = torch.randn(params.shape, generator=g).half()
    w = torch.randn(params.c, generator=g) if params.has_weight else None
    b = torch.randn(params.c, generator=g) if params.has_bias else None
    expected = _reference(x, w, b, params.eps)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    dyg = dy.cuda().contiguous(memory_format=torch.channels_last)
    wg = None if w is None else w.cuda()
    bg = None if b is None else b.cuda()
    for config in layernorm_2d_kernel_factory.configs(params, attr):
        kernel = layernorm_2d_kernel_factory.make_kernel(params, config, attr)
        kernel.compile()
        kernel.load(0)
        out = torch.full_like(xg, -42.0)
        kernel(out, xg, wg, bg)
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float().cpu(), expected, rtol=2e-3, atol=4e-3, msg=f"{params.encode()} {config}")
        kernel.unload()
    from dataclasses import replace

    params = replace(params, has_bias=False)  # the backward kernel never sees the bias
    if not layernorm_2d_bwd_is_supported(params):
        return
    ex_dx, ex_dw, _ = _reference_backward(x, dy, w, None, params.eps)
    ex_db = dy.float().sum(dim=(0, 2, 3))
    if ex_dw is None:
        ex_dw = (dy.float() * _reference(x, None, None, params.eps)).sum(dim=(0, 2, 3))
    for config in layernorm_2d_bwd_kernel_factory.configs(params, attr):
        kernel = layernorm_2d_bwd_kernel_factory.make_kernel(params, config, attr)
        kernel.compile()
        kernel.load(0)
        dx = torch.full_like(xg, -42.0)
        sums = torch.full((2, params.c), float("nan"), device="cuda")
        kernel(sums, dx, xg, dyg, wg)
        torch.cuda.synchronize()
        what = f"{params.encode()} {config}"
        torch.testing.assert_close(dx.float().cpu(), ex_dx, rtol=4e-3, atol=4e-3, msg=what)
        sums = sums.cpu()
        torch.testing.assert_close(sums[0], ex_dw, rtol=2e-3, atol=3e-2, msg=what)
        torch.testing.assert_close(sums[1], ex_db, rtol=2e-3, atol=3e-2, msg=what)
        kernel.unload()


def test_backward_falls_back_to_torch_operations(monkeypatch):
    """SPIO_LAYERNORM_BACKWARD=torch takes the torch-operation backward; same gradients."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 96, 6, 5, generator=g).half()
    dy = torch.randn(2, 96, 6, 5, generator=g).half()
    w, b = torch.randn(96, generator=g), torch.randn(96, generator=g)
    grads = []
    for mode in ("hip", "torch"):
        monkeypatch.setenv("SPIO_LAYERNORM_BACKWARD", mode)
        xg = x.cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
        wg, bg = w.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
        layernorm_2d(xg, wg, bg, 1e-6).backward(dy.cuda())
        grads.append((xg.grad.float().cpu(), wg.grad.cpu(), bg.grad.cpu()))
    for a, b_ in zip(*grads):
        torch.testing.assert_close(a, b_, rtol=4e-3, atol=2e-2)


@pytest.mark.parametrize("eps", [1e-6, 1e-3])
def test_layer_and_backward(eps):
    """eps = 1e-3 has a decimal point in its shortest form: the kernel's name must still be a symbol."""
    torch.manual_seed(0)
    layer = LayerNorm2d(96, eps=eps).cuda()
    with torch.no_grad():
        layer.weight.copy_(torch.randn(96))
        layer.bias.copy_(torch.randn(96))
    x = torch.randn(2, 96, 6, 5)
    dy = torch.randn(2, 96, 6, 5)
    xg = x.half().cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    y = layer(xg)
    y.backward(dy.half().cuda())
    xr = x.half().float().requires_grad_(True)
    wr = layer.weight.detach().cpu().clone().requires_grad_(True)
    br = layer.bias.detach().cpu().clone().requires_grad_(True)
    yr = _reference(xr, wr, br, eps)
    yr.backward(dy.half().float())
    torch.testing.assert_close(y.float().cpu(), yr.detach(), rtol=2e-3, atol=4e-3)
    torch.testing.assert_close(xg.grad.float().cpu(), xr.grad, rtol=4e-3, atol=4e-3)
    torch.testing.assert_close(layer.weight.grad.cpu(), wr.grad, rtol=2e-3, atol=2e-2)
    torch.testing.assert_close(layer.bias.grad.cpu(), br.grad, rtol=2e-3, atol=2e-2)


def test_opcheck_forward_and_backward_ops():
    """Schema, fake implementations (shapes, strides, dtypes) and autograd registration of both ops."""
    from spio_amd.functional.layernorm_2d_function import layernorm_2d_backward

    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 48, 5, 6, generator=g).half().cuda().contiguous(memory_format=torch.channels_last)
    dy = torch.randn(2, 48, 5, 6, generator=g).half().cuda().contiguous(memory_format=torch.channels_last)
    w, b = torch.randn(48, generator=g).cuda(), torch.randn(48, generator=g).cuda()
    torch.library.opcheck(layernorm_2d, (x.clone().requires_grad_(True), w.clone().requires_grad_(True),
                                         b.clone().requires_grad_(True), 1e-6))  # fmt: skip
    torch.library.opcheck(layernorm_2d_backward, (x, dy, w, 1e-6))
    torch.library.opcheck(layernorm_2d_backward, (x, dy, None, 1e-6))


def test_ops_replay_correctly_from_a_hip_graph():
    """Forward and backward ops captured once into a HIP graph and replayed three times on new
    data, with eager work and synchronisations between the replays; every replay must match the
    eager reference (both ops launch their own kernels only: no library reduction, no memset)."""
    from spio_amd.functional.layernorm_2d_function import layernorm_2d_backward

    g = torch.Generator().manual_seed(11)
    shape = (3, 192, 9, 10)
    x = torch.empty(shape, dtype=torch.float16, device="cuda").contiguous(memory_format=torch.channels_last)
    dy = torch.empty_like(x)
    w = torch.randn(192, generator=g).cuda()
    b = torch.randn(192, generator=g).cuda()

    def run():
        y = layernorm_2d(x, w, b, 1e-6)
        dx, sums = layernorm_2d_backward(x, dy, w, 1e-6)
        return y, dx, sums

    x.normal_(), dy.normal_()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # first use outside the capture: kernel compilation and loading
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = run()
    torch.cuda.current_stream().wait_stream(side)
    for trial in range(3):
        xt = (torch.randn(shape, generator=g) * 2 + 0.5).half()
        dyt = torch.randn(shape, generator=g).half()
        x.copy_(xt.cuda()), dy.copy_(dyt.cuda())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ex_y = _reference(xt, w.cpu(), b.cpu(), 1e-6)
        ex_dx, ex_dw, ex_db = _reference_backward(xt, dyt, w.cpu(), b.cpu(), 1e-6)
        msg = f"graph replay {trial}"
        torch.testing.assert_close(outs[0].float().cpu(), ex_y, rtol=2e-3, atol=4e-3, msg=msg)
        torch.testing.assert_close(outs[1].float().cpu(), ex_dx, rtol=4e-3, atol=4e-3, msg=msg)
        torch.testing.assert_close(outs[2][0].cpu(), ex_dw, rtol=2e-3, atol=3e-2, msg=msg)
        torch.testing.assert_close(outs[2][1].cpu(), ex_db, rtol=2e-3, atol=3e-2, msg=msg)

