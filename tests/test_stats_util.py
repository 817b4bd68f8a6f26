"""Known-answer tests taken from the reference's own tests
(tests/test_stats.py:9-52, tests/test_util.py:10-25) plus the byte counts of
the benchmark shapes.  CPU only."""

import pytest
import torch

from spio_amd.kernels import Conv2dGw8Params, Conv2dStats
from spio_amd.util import divup, next_relative_prime, to_channels_last, check_channels_last
from spio_amd.util.close import acc_depth_tolerances, assert_all_close_with_acc_depth
from spio_amd.util.env import env_var_is_true

P = Conv2dGw8Params(n=16, h=32, w=64, c=128, r=3, s=3)
NX = 16 * 32 * 64 * 128
NW = 128 * 8 * 3 * 3


def test_stats_fprop():
    st = Conv2dStats(P, output_names="output")
    assert st.bytes_read == (NX + NW) * 2
    assert st.bytes_written == NX * 2
    assert st.bytes == (NX + NW) * 2 + NX * 2
    assert st.macs == NX * 8 * 3 * 3
    assert st.accumulation_depths == [8 * 3 * 3]


def test_stats_input_grad():
    st = Conv2dStats(P, output_names="grad_input")
    assert st.bytes_read == (NX + NW) * 2
    assert st.bytes_written == NX * 2
    assert st.macs == NX * 8 * 3 * 3
    assert st.accumulation_depths == [8 * 3 * 3]


def test_stats_weight_grad():
    st = Conv2dStats(P, output_names="grad_weight")
    assert st.bytes_read == (NX + NX) * 2
    assert st.bytes_written == NW * 2
    assert st.grad_weight_bytes_written_fp32 == NW * 4
    assert st.macs == NX * 8 * 3 * 3
    assert st.accumulation_depths == [16 * 32 * 64]


def test_stats_bias_grad():
    assert Conv2dStats(P, output_names="grad_bias").accumulation_depths == [16 * 32 * 64]


def test_stats_bias_counts():
    pb = Conv2dGw8Params(n=16, h=32, w=64, c=128, r=3, s=3, has_bias=True)
    st = Conv2dStats(pb, output_names="output")
    assert st.bytes_read == (NX + NW + 128) * 2
    assert st.macs == NX * 72 + NX / 2
    assert st.op_byte == pytest.approx(2.0 * st.macs / st.bytes)


@pytest.mark.parametrize(
    "kw,expected",
    [
        (dict(n=32, c=64, h=56, w=56), 25_699_328),
        (dict(n=128, c=64, h=56, w=56), 102_769_664),
        (dict(n=128, c=128, h=28, w=28), 51_398_656),
        (dict(n=256, c=256, h=14, w=14, r=7, s=7, padding=3), 51_580_928),
    ],
)
def test_benchmark_shape_bytes(kw, expected):
    p = Conv2dGw8Params(**kw)
    assert Conv2dStats(p, output_names="output").bytes == expected
    assert Conv2dStats(p, output_names="grad_input").bytes == expected
    assert Conv2dStats(p, output_names="grad_weight").bytes == expected


def test_divup():
    assert divup(10, 3) == 4
    assert divup(9, 3) == 3
    assert divup(1, 16) == 1


def test_next_relative_prime():
    for n in range(1, 20):
        assert next_relative_prime(8 * n, 8) == 8 * n + 1
    assert [next_relative_prime(a, 8) for a in range(1, 8)] == [1, 3, 3, 5, 5, 7, 7]


def test_tolerance_rule():
    atol, rtol = acc_depth_tolerances(72)
    assert rtol == pytest.approx(1e-3)
    assert atol == pytest.approx(72 * 1.6 * 1.6 * 1.19e-7 * 3.5)
    e = torch.ones(4)
    assert_all_close_with_acc_depth(e + 5e-4, e, acc_depth=72)
    with pytest.raises(AssertionError):
        assert_all_close_with_acc_depth(e + 5e-3, e, acc_depth=72)
    with pytest.raises(AssertionError):
        assert_all_close_with_acc_depth(e * float("nan"), e, acc_depth=72)


def test_channels_last_helpers():
    x = torch.randn(2, 8, 3, 3)
    y, b, none = to_channels_last(x, torch.randn(8), None)
    assert y.is_contiguous(memory_format=torch.channels_last) and b.dim() == 1 and none is None
    assert to_channels_last(y)[0].data_ptr() == y.data_ptr()  # no copy when already channels_last
    check_channels_last([y, b, None])
    with pytest.raises(AssertionError):
        check_channels_last([x])


def test_env_truthiness(monkeypatch):
    for v, want in [("1", True), ("0", False), ("yes", True), ("T", True), ("no", False), ("-1", False), ("7", True)]:
        monkeypatch.setenv("SPIO_TEST_FLAG", v)
        assert env_var_is_true("SPIO_TEST_FLAG") is want
    monkeypatch.delenv("SPIO_TEST_FLAG")
    assert env_var_is_true("SPIO_TEST_FLAG") is False
