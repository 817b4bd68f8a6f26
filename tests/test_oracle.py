"""Pins the CPU oracle: three independent statements (torch, numpy loops, C)
must agree with each other and with closed forms that a plausible slip (wrong
sign of the padding offset, transposed filter index, flipped tap, wrong
grad_weight layout) would break.  CPU only."""

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import conv2d_gw8_oracle as oracle

TINY = [
    # n, c, h, w, r, s, py, px, bias
    (2, 8, 5, 6, 3, 3, 1, 1, True),
    (1, 16, 4, 5, 2, 3, 1, 0, False),
    (2, 8, 6, 4, 4, 1, 2, 0, True),
    (1, 8, 3, 3, 3, 3, 3, 2, False),  # padding larger than r-1: dgrad crops
    (1, 16, 7, 6, 5, 5, 2, 2, True),
]


def _args(case, seed=0, weight_init="randn"):
    n, c, h, w, r, s, py, px, bias = case
    return oracle.make_args(n, c, h, w, r, s, py, px, bias, seed=seed, weight_init=weight_init)


@pytest.mark.parametrize("case", TINY)
def test_three_statements_agree(case):
    n, c, h, w, r, s, py, px, _ = case
    x, wt, bias, dy = _args(case)
    y_t = oracle.fprop_torch(x, wt, bias, py, px)
    y_l = oracle.fprop_loops(x, wt, bias, py, px)
    y_c = c_oracle.fprop_c(x, wt, bias, py, px)
    assert torch.allclose(y_t, y_l, rtol=1e-5, atol=1e-4)
    assert torch.allclose(y_c, y_l, rtol=1e-5, atol=1e-4)

    dx_t, dw_t, db_t = oracle.grads_torch(x, wt, bias, dy, py, px)
    assert torch.allclose(dx_t, oracle.dgrad_loops(dy, wt, h, w, py, px), rtol=1e-5, atol=1e-4)
    assert torch.allclose(dx_t, c_oracle.dgrad_c(dy, wt, h, w, py, px), rtol=1e-5, atol=1e-4)
    assert torch.allclose(dw_t, oracle.wgrad_loops(x, dy, r, s, py, px), rtol=1e-5, atol=1e-3)
    assert torch.allclose(dw_t, c_oracle.wgrad_c(x, dy, r, s, py, px), rtol=1e-5, atol=1e-3)
    assert torch.allclose(db_t, c_oracle.dbias_c(dy), rtol=1e-5, atol=1e-3)
    assert torch.allclose(db_t, dy.float().sum(dim=(0, 2, 3)), rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("case", TINY)
def test_dgrad_is_fprop_with_flipped_transposed_filter(case):
    """The identity the kernel relies on (conv2d_gw8_kernel.py:73-83 in the reference)."""
    n, c, h, w, r, s, py, px, _ = case
    x, wt, bias, dy = _args(case)
    dx_t, _, _ = oracle.grads_torch(x, wt, None, dy, py, px)
    dx_f = oracle.dgrad_as_fprop_torch(dy, wt, r, s, py, px)
    assert dx_f.shape == dx_t.shape
    assert torch.allclose(dx_t, dx_f, rtol=1e-5, atol=1e-4)


def test_identity_filter_returns_input():
    """Centre-tap identity weights: y == x exactly (in every statement)."""
    n, c, h, w, r, s = 2, 16, 6, 7, 3, 3
    x = torch.randn(n, c, h, w).half()
    wt = torch.zeros(c, 8, r, s)
    for k in range(c):
        wt[k, k % 8, 1, 1] = 1.0
    wt = wt.half()
    for y in (oracle.fprop_torch(x, wt, None, 1, 1), oracle.fprop_loops(x, wt, None, 1, 1),
              c_oracle.fprop_c(x, wt, None, 1, 1)):  # fmt: skip
        assert torch.equal(y, x.float())


def test_shift_filter_direction():
    """A single off-centre tap shifts the image the way y[p,q] = x[p+r-py, q+s-px] says."""
    x = torch.arange(1 * 8 * 5 * 5, dtype=torch.float32).reshape(1, 8, 5, 5).half()
    wt = torch.zeros(8, 8, 3, 3)
    for k in range(8):
        wt[k, k, 0, 2] = 1.0  # tap r=0, s=2 with pad 1: y[p,q] = x[p-1, q+1]
    wt = wt.half()
    expect = torch.zeros(1, 8, 5, 5)
    expect[:, :, 1:, :-1] = x.float()[:, :, :-1, 1:]
    for y in (oracle.fprop_torch(x, wt, None, 1, 1), oracle.fprop_loops(x, wt, None, 1, 1),
              c_oracle.fprop_c(x, wt, None, 1, 1)):  # fmt: skip
        assert torch.equal(y, expect)


def test_all_ones_counts_valid_taps():
    """x = w = 1: y = 8 * (number of taps inside the image), a border pattern."""
    n, c, h, w, r, s, py, px = 1, 8, 5, 4, 3, 3, 1, 1
    x = torch.ones(n, c, h, w).half()
    wt = torch.ones(c, 8, r, s).half()
    rows = torch.tensor([min(p + r - py, h) - max(p - py, 0) for p in range(h)]).float()
    cols = torch.tensor([min(q + s - px, w) - max(q - px, 0) for q in range(w)]).float()
    expect = (8 * rows[:, None] * cols[None, :]).expand(n, c, h, w)
    assert torch.equal(oracle.fprop_torch(x, wt, None, py, px), expect)
    assert torch.equal(c_oracle.fprop_c(x, wt, None, py, px), expect)


def test_one_by_one_is_block_diagonal_matmul():
    """R = S = 1: each pixel is multiplied by a block-diagonal 8x8-per-group matrix."""
    n, c, h, w = 2, 24, 3, 4
    x, wt, bias, _ = oracle.make_args(n, c, h, w, 1, 1, 0, 0, True, seed=3, weight_init="randn")
    full = torch.zeros(c, c)
    for k in range(c):
        g = k // 8
        full[k, 8 * g : 8 * g + 8] = wt[k, :, 0, 0].float()
    expect = torch.einsum("kc,nchw->nkhw", full, x.float()) + bias[None, :, None, None]
    assert torch.allclose(oracle.fprop_torch(x, wt, bias, 0, 0), expect, rtol=1e-5, atol=1e-5)
    assert torch.allclose(c_oracle.fprop_c(x, wt, bias, 0, 0), expect, rtol=1e-5, atol=1e-5)


def test_zero_weights_give_bias():
    x, wt, bias, _ = oracle.make_args(2, 16, 4, 4, 3, 3, 1, 1, True, seed=4)
    y = oracle.fprop_torch(x, torch.zeros_like(wt), bias, 1, 1)
    assert torch.equal(y, bias[None, :, None, None].expand_as(y))
    assert torch.equal(c_oracle.fprop_c(x, torch.zeros_like(wt), bias, 1, 1), y)


@pytest.mark.parametrize("case", TINY)
def test_adjoint_identities(case):
    """<conv(x), dy> == <x, dgrad(dy)> == <w, wgrad(x, dy)> (conv is bilinear)."""
    n, c, h, w, r, s, py, px, _ = case
    x, wt, _b, dy = _args(case, seed=7)
    y = c_oracle.fprop_c(x, wt, None, py, px).double()
    lhs = float((y * dy.double()).sum())
    dx = c_oracle.dgrad_c(dy, wt, h, w, py, px).double()
    dw = c_oracle.wgrad_c(x, dy, r, s, py, px).double()
    assert lhs == pytest.approx(float((dx * x.double()).sum()), rel=1e-5, abs=1e-3)
    assert lhs == pytest.approx(float((dw * wt.double()).sum()), rel=1e-5, abs=1e-3)


def test_wgrad_layout_single_element():
    """One non-zero x and one non-zero dy light up exactly one (k, c, r, s)."""
    n, c, h, w, r, s, py, px = 1, 16, 5, 5, 3, 3, 1, 1
    x = torch.zeros(n, c, h, w).half()
    dy = torch.zeros(n, c, h, w).half()
    x[0, 8 + 3, 2, 4] = 2.0  # group 1, channel-in-group 3
    dy[0, 8 + 5, 3, 3] = 3.0  # group 1, out channel 13: r = 2-3+1 = 0, s = 4-3+1 = 2
    for dw in (c_oracle.wgrad_c(x, dy, r, s, py, px), oracle.wgrad_loops(x, dy, r, s, py, px),
               oracle.grads_torch(x, torch.zeros(c, 8, r, s).half(), None, dy, py, px)[1]):  # fmt: skip
        nz = torch.nonzero(dw)
        assert nz.tolist() == [[13, 3, 0, 2]]
        assert float(dw[13, 3, 0, 2]) == 6.0


def test_c_oracle_half_conversion_all_bit_patterns():
    """The C half->float conversion agrees with numpy for every finite fp16 bit pattern."""
    bits = np.arange(65536, dtype=np.uint16)
    halves = bits.view(np.float16)
    finite = np.isfinite(halves)
    x = torch.from_numpy(halves[finite].astype(np.float32)).half()
    count = x.numel()
    pad = (-count) % 8
    x = torch.cat([x, torch.zeros(pad).half()]).reshape(1, 8, -1, 1)
    wt = torch.zeros(8, 8, 1, 1)
    for k in range(8):
        wt[k, k, 0, 0] = 1.0
    y = c_oracle.fprop_c(x, wt.half(), None, 0, 0)
    assert torch.equal(y, x.float())


def test_make_args_is_seeded_and_fp16_channels_last():
    a = oracle.make_args(2, 16, 5, 5, 3, 3, 1, 1, True, seed=5)
    b = oracle.make_args(2, 16, 5, 5, 3, 3, 1, 1, True, seed=5)
    for s, t in zip(a, b):
        assert torch.equal(s, t)
    assert a[0].dtype == torch.float16 and a[0].is_contiguous(memory_format=torch.channels_last)
    assert a[2].dtype == torch.float32
    assert float(a[0].abs().max()) <= 3.0
    fan_in = 8 * 9
    assert float(a[1].abs().max()) <= (1.0 / fan_in) ** 0.5 + 1e-3  # kaiming-uniform bound
