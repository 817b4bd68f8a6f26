"""The benchmark configurations at their full sizes, through the operator (tuned kernels are
used when a record exists, else the first configuration), against the fp32 CPU oracle, plus
size-independent properties (bilinearity / adjoint identities evaluated from the GPU results) and
the ConvNeXt-shaped network.  GPU only."""

import pytest
import torch

from spio_amd.convnext_gw8 import ConvNeXtGw8
from helpers import to_gpu
from oracle import conv2d_gw8_oracle as oracle
from spio_amd.functional import conv2d_gw8
from spio_amd.kernels import Conv2dGw8Params, Conv2dStats
from spio_amd.layers import Conv2dGw8
from spio_amd.transform import transform

pytestmark = pytest.mark.gpu

CONFIGS = {
    "cfg1": (Conv2dGw8Params(n=32, c=64, h=56, w=56, padding=1), 0),
    "cfg2": (Conv2dGw8Params(n=128, c=128, h=28, w=28, padding=1), 1),
    "cfg3": (Conv2dGw8Params(n=256, c=256, h=14, w=14, padding=3, r=7, s=7), 2),
    "target": (Conv2dGw8Params(n=128, c=64, h=56, w=56, padding=1), 0),
}


def _run(params, seed):
    x, w, _b, dy = oracle.make_args(params.n, params.c, params.h, params.w, params.r, params.s,
                                    params.padding_h, params.padding_w, False, seed, weight_init="kaiming")  # fmt: skip
    xg, wg, dyg = to_gpu(x).requires_grad_(True), to_gpu(w).requires_grad_(True), to_gpu(dy)
    y = conv2d_gw8(xg, wg, None, stride=1, padding_y=params.padding_h, padding_x=params.padding_w,
                   groups=params.groups)  # fmt: skip
    dx, dw, _none = torch.ops.spio.conv2d_gw8_backward(xg.detach(), wg.detach(), None, dyg, params.padding_h,
                                                       params.padding_w, True, True, False)  # fmt: skip
    torch.cuda.synchronize()
    return x, w, dy, y.detach(), dx, dw


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size_against_oracle(name):
    """North-star tolerance (rel 2e-3 / atol 1e-2 on fp16 outputs) and the reference's
    accumulation-depth tolerance, at the benchmark size."""
    params, seed = CONFIGS[name]
    x, w, dy, y, dx, dw = _run(params, seed)
    depth = Conv2dStats(params, output_names=["output", "grad_input", "grad_weight"]).accumulation_depths
    y_e = oracle.fprop_torch(x, w, None, params.padding_h, params.padding_w)
    oracle.check_close(y, y_e, what=f"{name} fprop (north-star tolerance)")
    oracle.check_close(y, y_e, acc_depth=depth[0], what=f"{name} fprop")
    dx_e, dw_e, _ = oracle.grads_torch(x, w, None, dy, params.padding_h, params.padding_w)
    oracle.check_close(dx, dx_e, what=f"{name} dgrad (north-star tolerance)")
    oracle.check_close(dx, dx_e, acc_depth=depth[1], what=f"{name} dgrad")
    assert dw.dtype == torch.float32
    oracle.check_close(dw, dw_e, acc_depth=depth[2], what=f"{name} wgrad")


def test_target_size_with_separate_backward_kernels(monkeypatch):
    """The recorded times make the backward op pick the fused kernel at the target size; with
    fusing switched off the separate data- and weight-gradient kernels must give the same answer."""
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", "0")
    params, seed = CONFIGS["target"]
    x, w, dy, _y, dx, dw = _run(params, seed)
    depth = Conv2dStats(params, output_names=["grad_input", "grad_weight"]).accumulation_depths
    dx_e, dw_e, _ = oracle.grads_torch(x, w, None, dy, params.padding_h, params.padding_w)
    oracle.check_close(dx, dx_e, acc_depth=depth[0], what="target dgrad (separate)")
    oracle.check_close(dw, dw_e, acc_depth=depth[1], what="target wgrad (separate)")


@pytest.mark.parametrize("name", ["cfg2", "cfg3"])
def test_adjoint_identities_from_gpu_results(name):
    """<conv(x), dy> == <x, dgrad(dy)> == <w, wgrad(x, dy)>, evaluated in fp64 from what the
    kernels returned.  y and dx are rounded to fp16, so the identities hold to ~1e-3 relative."""
    params, seed = CONFIGS[name]
    x, w, dy, y, dx, dw = _run(params, seed)
    lhs = float((y.double().cpu() * dy.double()).sum())
    via_dx = float((dx.double().cpu() * x.double()).sum())
    via_dw = float((dw.double().cpu() * w.double()).sum())
    scale = float((y.double().cpu().abs() * dy.double().abs()).sum())
    assert abs(lhs - via_dx) <= 2e-3 * scale * 1e-1
    assert abs(lhs - via_dw) <= 2e-3 * scale * 1e-1
    assert abs(via_dx - via_dw) <= 2e-3 * scale * 1e-1


def test_forward_is_linear_in_the_input_at_full_size():
    """conv(a + b) == conv(a) + conv(b) up to the output rounding, at the benchmark size."""
    params, seed = CONFIGS["target"]
    a, w, _b, _dy = oracle.make_args(params.n, params.c, params.h, params.w, 3, 3, 1, 1, False, seed)
    b = oracle.make_args(params.n, params.c, params.h, params.w, 3, 3, 1, 1, False, seed + 1)[0]
    ag, bg, wg = to_gpu(a), to_gpu(b), to_gpu(w)
    sg = (ag.float() + bg.float()).half()  # the sum itself is rounded: compare against conv of that
    call = lambda t: conv2d_gw8(t, wg, None, 1, 1, 1, 1, params.groups).float()
    lhs = call(sg)
    rhs = call(ag) + call(bg)
    # |x| <= 6, 72 products with |w| <= 0.12: the rounding of s and of the three outputs stays
    # far below this bound
    assert float((lhs - rhs).abs().max()) < 0.05
    assert float((lhs - rhs).abs().mean()) < 2e-3


@pytest.mark.parametrize("n", [1, 2, 4, 8, 16, 32, 64, 128, 256, 512])
def test_batch_sweep_forward(n):
    """Forward at C=64, 56x56 for every batch size of the sweep configuration."""
    params = Conv2dGw8Params(n=n, c=64, h=56, w=56, padding=1)
    x, w, _b, _dy = oracle.make_args(n, 64, 56, 56, 3, 3, 1, 1, False, 0, weight_init="kaiming")
    y = conv2d_gw8(to_gpu(x), to_gpu(w), None, 1, 1, 1, 1, 8)
    expected = oracle.fprop_torch(x, w, None, 1, 1)
    oracle.check_close(y, expected, acc_depth=72, what=params.encode())
    oracle.check_close(y, expected, what=params.encode() + " (north-star tolerance)")


@pytest.mark.parametrize("n", [64, 256])
def test_batch_sweep_backward(n):
    """Backward at the sweep batch sizes that no other configuration covers."""
    params = Conv2dGw8Params(n=n, c=64, h=56, w=56, padding=1)
    x, w, dy, _y, dx, dw = _run(params, 0)
    depth = Conv2dStats(params, output_names=["grad_input", "grad_weight"]).accumulation_depths
    dx_e, dw_e, _ = oracle.grads_torch(x, w, None, dy, 1, 1)
    oracle.check_close(dx, dx_e, acc_depth=depth[0], what=f"N={n} dgrad")
    oracle.check_close(dw, dw_e, acc_depth=depth[1], what=f"N={n} wgrad")


@pytest.mark.parametrize("c,hw", [(96, 56), (192, 28), (384, 14), (768, 7)])
def test_network_conv_shapes_at_full_batch_with_bias(c, hw):
    """The four gw8 convolution shapes of the network configuration at batch 128, with bias,
    forward and backward through the operators with the recorded configurations."""
    params = Conv2dGw8Params(n=128, c=c, h=hw, w=hw, padding=1, has_bias=True)
    x, w, b, dy = oracle.make_args(128, c, hw, hw, 3, 3, 1, 1, True, 3, weight_init="kaiming")
    xg, wg, bg, dyg = to_gpu(x), to_gpu(w), to_gpu(b), to_gpu(dy)
    y = conv2d_gw8(xg, wg, bg, stride=1, padding_y=1, padding_x=1, groups=c // 8)
    dx, dw, db = torch.ops.spio.conv2d_gw8_backward(xg, wg, bg, dyg, 1, 1, True, True, True)
    torch.cuda.synchronize()
    depth = Conv2dStats(params, output_names=["output", "grad_input", "grad_weight", "grad_bias"]).accumulation_depths
    oracle.check_close(y, oracle.fprop_torch(x, w, b, 1, 1), acc_depth=depth[0], what=f"{params.encode()} fprop")
    dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, 1, 1)
    oracle.check_close(dx, dx_e, acc_depth=depth[1], what=f"{params.encode()} dgrad")
    oracle.check_close(dw, dw_e, acc_depth=depth[2], what=f"{params.encode()} wgrad")
    oracle.check_close(db, db_e, acc_depth=depth[3], what=f"{params.encode()} grad_bias")


def test_convnext_shaped_network_logits():
    """The network of the fifth configuration: logits of the fp16 GPU model with Conv2dGw8
    layers against the same weights in fp32 on the CPU with nn.Conv2d(groups=C/8).  Batch 4
    keeps the CPU side to seconds; every gw8 convolution shape of the full-batch run occurs."""
    torch.manual_seed(3)
    cpu_model = ConvNeXtGw8().eval()
    images = torch.randn(4, 3, 224, 224).half().float()
    with torch.no_grad():
        want = cpu_model(images)
    gpu_model = transform(ConvNeXtGw8().eval())
    gpu_model.load_state_dict(cpu_model.state_dict())
    assert sum(isinstance(m, Conv2dGw8) for m in gpu_model.modules()) == 18
    gpu_model = gpu_model.cuda().to(memory_format=torch.channels_last)
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.float16):
        got = gpu_model(images.cuda().contiguous(memory_format=torch.channels_last))
    got = got.float().cpu()
    # 18 residual blocks in fp16 against fp32: logits are O(1); agree to a few 1e-2 and rank alike
    assert float((got - want).abs().max()) < 0.08 * max(1.0, float(want.abs().max()))
    assert torch.equal(got.argmax(dim=1), want.argmax(dim=1))
    # ... and a wrong convolution would show: zeroing one conv's weights moves the logits
    first = next(m for m in gpu_model.modules() if isinstance(m, Conv2dGw8))
    with torch.no_grad():
        saved = first.weight.clone()
        first.weight.zero_()
        with torch.autocast(device_type="cuda", dtype=torch.float16):
            moved = gpu_model(images.cuda().contiguous(memory_format=torch.channels_last)).float().cpu()
        first.weight.copy_(saved)
    assert float((moved - want).abs().max()) > 10 * float((got - want).abs().max())


def test_convnext_shaped_network_with_layernorm_kernels():
    """The same network built directly from Conv2dGw8 and the LayerNorm2d kernel layer, under fp16
    autocast as the benchmark runs it, against the fp32 CPU model."""
    from spio_amd.layers import LayerNorm2d

    torch.manual_seed(3)
    cpu_model = ConvNeXtGw8().eval()
    images = torch.randn(4, 3, 224, 224).half().float()
    with torch.no_grad():
        want = cpu_model(images)
    gpu_model = ConvNeXtGw8(make_conv=lambda d: Conv2dGw8(d, d, 3, padding=1, groups=d // 8), norm2d=LayerNorm2d)
    gpu_model.load_state_dict(cpu_model.state_dict())
    gpu_model = gpu_model.eval().cuda().to(memory_format=torch.channels_last)
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.float16):
        got = gpu_model(images.cuda().contiguous(memory_format=torch.channels_last))
    got = got.float().cpu()
    assert float((got - want).abs().max()) < 0.08 * max(1.0, float(want.abs().max()))
    assert torch.equal(got.argmax(dim=1), want.argmax(dim=1))


def test_convnext_shaped_network_at_batch_128():
    """The configuration the benchmark times: batch 128, Conv2dGw8 and LayerNorm2d kernel layers,
    fp16 autocast, channels_last.  The network treats every image on its own, so the logits of
    the first 8 images of the batch are compared with the fp32 CPU model run on those 8 images."""
    from spio_amd.layers import LayerNorm2d

    torch.manual_seed(3)
    cpu_model = ConvNeXtGw8().eval()
    images = torch.randn(128, 3, 224, 224, generator=torch.Generator().manual_seed(3)).half()
    with torch.no_grad():
        want = cpu_model(images[:8].float())
    gpu_model = ConvNeXtGw8(make_conv=lambda d: Conv2dGw8(d, d, 3, padding=1, groups=d // 8),
                            norm2d=lambda d: LayerNorm2d(d, eps=1e-5))  # fmt: skip
    gpu_model.load_state_dict(cpu_model.state_dict())
    gpu_model = gpu_model.eval().cuda().to(memory_format=torch.channels_last)
    with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.float16):
        got = gpu_model(images.cuda().contiguous(memory_format=torch.channels_last))
    assert got.shape == (128, 1000)
    got8 = got[:8].float().cpu()
    assert float((got8 - want).abs().max()) < 0.08 * max(1.0, float(want.abs().max()))
    assert torch.equal(got8.argmax(dim=1), want.argmax(dim=1))
    assert torch.isfinite(got).all()


def _repeat_images(t, rep):
    """[n, C, H, W] -> [n * rep, C, H, W] on the GPU in channels_last memory, the n images repeated."""
    nhwc = t.cuda().permute(0, 2, 3, 1).contiguous()
    return nhwc.repeat(rep, 1, 1, 1).permute(0, 3, 1, 2)


def _blocks_equal_first(t, rep):
    v = t.permute(0, 2, 3, 1).reshape(rep, -1)
    return all(bool((v[i:i + 64] == v[0:1]).all()) for i in range(0, rep, 64))


@pytest.mark.parametrize("mode", ["1", "0"])
def test_tensors_beyond_4_gib(monkeypatch, mode):
    """N = 11000 images of 64 channels, 56x56: every activation tensor holds 2.2e9 elements in
    4.4 GB, past what 32-bit element indices and byte offsets reach.  The batch is 8 seeded
    images repeated 1375 times: the first and last 8 outputs and input gradients are checked
    against the oracle, every other block of 8 must equal the first bit for bit, and the weight
    and bias gradients must be 1375 times the oracle's for the 8 images.  With the fused backward
    kernel and with the separate ones."""
    monkeypatch.setenv("SPIO_FUSED_BACKWARD", mode)
    rep = 1375
    x, w, b, dy = oracle.make_args(8, 64, 56, 56, 3, 3, 1, 1, True, 5, weight_init="kaiming")
    y_e = oracle.fprop_torch(x, w, b, 1, 1)
    dx_e, dw_e, db_e = oracle.grads_torch(x, w, b, dy, 1, 1)
    xb, dyb = _repeat_images(x, rep), _repeat_images(dy, rep)
    assert xb.numel() > 2**31 and xb.is_contiguous(memory_format=torch.channels_last)
    wg, bg = to_gpu(w), to_gpu(b)
    y = conv2d_gw8(xb, wg, bg, stride=1, padding_y=1, padding_x=1, groups=8)
    oracle.check_close(y[:8], y_e, what="fprop, first images")
    oracle.check_close(y[-8:], y_e, what="fprop, last images")
    assert _blocks_equal_first(y, rep)
    del y
    dx, dw, db = torch.ops.spio.conv2d_gw8_backward(xb, wg, bg, dyb, 1, 1, True, True, True)
    oracle.check_close(dx[:8], dx_e, what="dgrad, first images")
    oracle.check_close(dx[-8:], dx_e, what="dgrad, last images")
    assert _blocks_equal_first(dx, rep)
    for got, expected, name in ((dw, dw_e * rep, "grad_weight"), (db, db_e * rep, "grad_bias")):
        err = (got.cpu().float() - expected).abs().max().item()
        assert err <= 1e-3 * expected.abs().max().item(), f"{name}: {err}"


def test_layernorm_tensors_beyond_4_gib():
    """LayerNorm2d forward and backward on 11000 images of 96 channels, 56x56 (3.3e9 elements,
    6.6 GB per tensor): 8 seeded images repeated; blocks equal the first one, the first block is
    checked against torch in fp32, the channel sums are 1375 times those of the 8 images."""
    from spio_amd.functional import layernorm_2d
    from spio_amd.functional.layernorm_2d_function import layernorm_2d_backward

    rep = 1375
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(8, 96, 56, 56, generator=g) * 2 + 0.5).half()
    dy = torch.randn(8, 96, 56, 56, generator=g).half()
    w, b = torch.randn(96, generator=g), torch.randn(96, generator=g)
    xr = x.float().requires_grad_(True)
    wr = w.clone().requires_grad_(True)
    y_e = torch.nn.functional.layer_norm(xr.permute(0, 2, 3, 1), (96,), wr, b, 1e-6).permute(0, 3, 1, 2)
    y_e.backward(dy.float())
    xb, dyb = _repeat_images(x, rep), _repeat_images(dy, rep)
    assert xb.numel() > 2**31
    y = layernorm_2d(xb, w.cuda(), b.cuda(), 1e-6)
    torch.testing.assert_close(y[:8].float().cpu(), y_e.detach(), rtol=2e-3, atol=4e-3)
    assert _blocks_equal_first(y, rep)
    del y
    dx, sums = layernorm_2d_backward(xb, dyb, w.cuda(), 1e-6)
    torch.testing.assert_close(dx[:8].float().cpu(), xr.grad, rtol=4e-3, atol=4e-3)
    assert _blocks_equal_first(dx, rep)
    sums = sums.cpu()
    for got, expected in ((sums[0], wr.grad * rep), (sums[1], dy.float().sum(dim=(0, 2, 3)) * rep)):
        assert (got - expected).abs().max().item() <= 1e-3 * expected.abs().max().item()
