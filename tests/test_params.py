"""Conv2dGw8Params: encode/decode, derived shapes, validation, layer matching.  CPU only."""

import pytest
import torch
from torch import nn

from spio_amd.kernels import Conv2dGw8Params
from spio_amd.layers import Conv2dGw8, make_conv2d


def test_encode_literal_and_round_trip():
    p = Conv2dGw8Params(n=32, c=64, h=56, w=56)
    assert p.encode() == "32n_64c_56h_56w_1py_1px_3r_3s_nb"
    q = Conv2dGw8Params(n=4, c=128, h=32, w=31, padding=(2, 0), r=4, s=1, has_bias=True)
    assert q.encode() == "4n_128c_32h_31w_2py_0px_4r_1s_b"
    d = Conv2dGw8Params.decode(q.encode())
    assert d == q and d.padding == (2, 0)
    assert Conv2dGw8Params.decode(p.encode()).encode() == p.encode()
    with pytest.raises(ValueError):
        Conv2dGw8Params.decode("32n_64c")


def test_derived_shapes():
    p = Conv2dGw8Params(n=2, c=16, h=10, w=12, padding=(2, 0), r=4, s=1)
    assert (p.p, p.q) == (10 + 4 - 4 + 1, 12)
    assert p.output_shape == (2, 16, 11, 12)
    assert p.weight_shape == (16, 8, 4, 1)
    assert p.bias_shape == (16,)
    assert p.groups == 2 and p.k == 16 and p.kernel_size == (4, 1)
    assert (p.transpose_padding_h, p.transpose_padding_w) == (1, 0)
    big = Conv2dGw8Params(n=1, c=128, h=64, w=64, padding=7)
    assert big.transpose_padding_h == -5 and big.p == 76


def test_validate():
    assert Conv2dGw8Params(n=1, c=8, h=1, w=1, padding=1).is_valid()
    assert not Conv2dGw8Params(n=1, c=12, h=8, w=8).is_valid()
    assert not Conv2dGw8Params(n=0, c=8, h=8, w=8).is_valid()
    assert not Conv2dGw8Params(n=1, c=8, h=8, w=8, r=8, s=3).is_valid()
    assert not Conv2dGw8Params(n=1, c=8, h=2, w=2, padding=0, r=3, s=3).is_valid()  # empty output
    assert Conv2dGw8Params(n=1, c=8, h=8, w=8, r=7, s=7, padding=3).is_valid()  # extension beyond 5


def test_from_tensors():
    x = torch.zeros(2, 16, 5, 6)
    w = torch.zeros(16, 8, 3, 3)
    p = Conv2dGw8Params.from_tensors(x, w, torch.zeros(16), (1, 1))
    assert p == Conv2dGw8Params(n=2, c=16, h=5, w=6, padding=(1, 1), has_bias=True)
    with pytest.raises(AssertionError):
        Conv2dGw8Params.from_tensors(x, torch.zeros(16, 4, 3, 3), None)
    with pytest.raises(AssertionError):
        Conv2dGw8Params.from_tensors(x, torch.zeros(32, 8, 3, 3), None)
    with pytest.raises(AssertionError):
        Conv2dGw8Params.from_tensors(x, w, torch.zeros(8), 1)


def test_match_args_truth_table():
    m = Conv2dGw8.match_args
    assert m(64, 64, 3, groups=8)
    assert m(64, 64, (5, 1), stride=(1, 1), dilation=(1, 1), groups=8)
    assert not m(64, 128, 3, groups=8)  # in != out
    assert not m(64, 64, 3, groups=4)  # group width 16
    assert not m(64, 64, 3, groups=64)  # depthwise
    assert not m(64, 64, 7, groups=8)  # kernel size > 5
    assert not m(64, 64, 3, stride=2, groups=8)
    assert not m(64, 64, 3, dilation=2, groups=8)
    assert not m(64, 64, 3, groups=8, padding_mode="reflect")


def test_match_make_and_from_torch_module():
    conv = nn.Conv2d(32, 32, 3, padding=1, groups=4)
    assert Conv2dGw8.match(conv)
    mod = Conv2dGw8.from_torch_module(conv)
    assert isinstance(mod, Conv2dGw8) and not Conv2dGw8.match(mod)
    assert mod.weight is conv.weight and mod.bias is conv.bias  # shared, not copied
    assert mod.padding == (1, 1) and mod.groups == 4
    with pytest.raises(ValueError):
        Conv2dGw8.from_torch_module(nn.Conv2d(32, 32, 3, groups=1))
    assert make_conv2d(32, 32, 3, groups=4, padding=1) is not None
    assert make_conv2d(32, 64, 3, groups=4) is None


def test_op_rejects_cpu_and_bad_dtypes():
    from spio_amd.functional import conv2d_gw8

    x = torch.zeros(1, 8, 4, 4, dtype=torch.float16)
    w = torch.zeros(8, 8, 3, 3, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        conv2d_gw8(x, w, None, 1, 1, 1, 1, 1)
    with pytest.raises(AssertionError):
        conv2d_gw8(x.float(), w, None, 1, 1, 1, 1, 1)
    with pytest.raises(AssertionError):
        conv2d_gw8(x, w, None, 2, 1, 1, 1, 1)  # stride
    with pytest.raises(AssertionError):
        conv2d_gw8(x, w, None, 1, 1, 1, 1, 2)  # groups != C // 8


def test_fake_impl_shapes():
    """FakeTensor propagation (what torch.compile uses) needs no GPU."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    import spio_amd.functional  # noqa: F401

    with FakeTensorMode():
        x = torch.empty(2, 16, 9, 7, dtype=torch.float16)
        w = torch.empty(16, 8, 3, 3, dtype=torch.float16)
        b = torch.empty(16, dtype=torch.float32)
        y = torch.ops.spio.conv2d_gw8(x, w, b, 1, 1, 0, 1, 2)
        assert tuple(y.shape) == (2, 16, 9, 5) and y.dtype == torch.float16
        assert y.is_contiguous(memory_format=torch.channels_last)
        dx, dw, db = torch.ops.spio.conv2d_gw8_backward(x, w, b, y, 1, 0, True, True, True)
        assert dx.shape == x.shape and dw.shape == w.shape and db.shape == b.shape
        assert dw.dtype == torch.float32 and db.dtype == torch.float32
        dx, dw, db = torch.ops.spio.conv2d_gw8_backward(x, w, b, y, 1, 0, False, True, False)
        assert dx is None and db is None
