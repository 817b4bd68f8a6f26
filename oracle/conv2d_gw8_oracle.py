"""CPU restatement of the conv2d_gw8 contract -- TEST INFRASTRUCTURE ONLY.

This file states, on the CPU, what the reference's GPU path computes, so that
the HIP kernels can be compared with it.  It is never imported by the product
package; the product has no CPU fallback.

What the reference computes (group g = k // 8, zero outside the input):
  fprop  y[n,k,p,q]  = bias[k] + sum_{c<8,r,s} x[n,8g+c,p+r-py,q+s-px] * w[k,c,r,s]
         fp32 accumulation of fp16 products, bias added in fp32, one rounding
         to fp16 at the store (spio/src/conv2d_gw8.cu:27-33,139,160-166,213-220).
  dgrad  dx[n,8g+c,h,w] = sum_{j<8,r,s} dy[n,8g+j,h-r+py,w-s+px] * w[8g+j,c,r,s]
         the same kernel run on dy with the flipped, group-transposed filter
         and padding (R-1-py, S-1-px)
         (spio/kernels/conv2d_gw8_kernel.py:73-83; spio/src/conv2d_gw8.cu:99-102).
  wgrad  dw[k,c,r,s] = sum_{n,p,q} x[n,8g+c,p+r-py,q+s-px] * dy[n,k,p,q], kept in fp32
         (spio/src/conv2d_gw8_wgrad.cu:92-225).
  dbias  db[k] = sum_{n,p,q} dy[n,k,p,q] in fp32
         (spio/functional/conv2d_gw8_function.py:134-136).

The reference's own tests use exactly the torch formulation below as their
oracle: F.conv2d in fp32 on the fp16-rounded tensors
(spio/reflection/conv2d_gw8_reflection.py:31,43,101,123;
spio/src_tests/run_test.py:43-50, 91-102).  `*_torch` functions follow it.
`*_loops` functions are an independent 7-loop numpy statement for tiny
shapes, and oracle/conv2d_gw8_oracle.c is an independent C statement for
medium shapes; tests/test_oracle.py checks the three against each other and
against closed forms, so a slip in any one of them (sign of the padding
offset, transposed filter index, flipped tap) fails.

Pinned by: tests/test_oracle.py (closed forms, cross-checks, adjoint
identities) and tests/test_stats_util.py (the reference's known-answer tests).
No function here is "parity unpinned" except kernel sizes 6 and 7, which the
reference rejects (spio/kernels/conv2d_gw8_params.py:137-138): for them only
torch's conv2d and the loop/C statements pin the result.
"""

import numpy as np
import torch
import torch.nn.functional as F

GROUP_WIDTH = 8

# Tolerance stated for this build: rel 2e-3 / atol 1e-2 on fp16 outputs.
NORTH_STAR_RTOL = 2e-3
NORTH_STAR_ATOL = 1e-2


# ----------------------------------------------------------------------------
# torch formulation (the reference's own test oracle)
# ----------------------------------------------------------------------------
def fprop_torch(x16, w16, bias32, py, px):
    """fp32 result of the forward conv on fp16-rounded operands (not yet rounded to fp16)."""
    groups = x16.shape[1] // GROUP_WIDTH
    return F.conv2d(
        x16.float().cpu(), w16.float().cpu(), None if bias32 is None else bias32.float().cpu(),
        stride=1, padding=(py, px), dilation=1, groups=groups,
    )  # fmt: skip


def grads_torch(x16, w16, bias32, dy16, py, px):
    """(dx, dw, db) in fp32 via autograd of the fp32 forward (run_test.py:91-102)."""
    x = x16.float().cpu().detach().requires_grad_(True)
    w = w16.float().cpu().detach().requires_grad_(True)
    b = None if bias32 is None else bias32.float().cpu().detach().requires_grad_(True)
    groups = x.shape[1] // GROUP_WIDTH
    y = F.conv2d(x, w, b, stride=1, padding=(py, px), dilation=1, groups=groups)
    leaves = [x, w] + ([b] if b is not None else [])
    grads = torch.autograd.grad(y, leaves, dy16.float().cpu())
    dx, dw = grads[0], grads[1]
    db = grads[2] if b is not None else dy16.float().cpu().sum(dim=(0, 2, 3))
    return dx, dw, db


def dgrad_as_fprop_torch(dy16, w16, r, s, py, px):
    """dgrad written the way the kernel runs it: forward conv of dy with the
    flipped, group-transposed filter and the transposed padding; negative
    padding crops (conv2d_gw8_kernel.py:73-83)."""
    k = w16.shape[0]
    g = k // GROUP_WIDTH
    w = w16.float().cpu().reshape(g, GROUP_WIDTH, GROUP_WIDTH, r, s)  # [g][j][c][r][s]
    wt = w.permute(0, 2, 1, 3, 4).flip(3, 4).reshape(k, GROUP_WIDTH, r, s)  # [g][c][j] flipped
    tpy, tpx = r - 1 - py, s - 1 - px
    dy = dy16.float().cpu()
    # F.conv2d accepts only non-negative padding: pad (or crop) by hand.
    dy = F.pad(dy, (tpx, tpx, tpy, tpy))
    return F.conv2d(dy, wt, None, stride=1, padding=0, groups=g)


# ----------------------------------------------------------------------------
# independent numpy loops (tiny shapes only)
# ----------------------------------------------------------------------------
def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def fprop_loops(x16, w16, bias32, py, px):
    x, w = _np(x16), _np(w16)
    n_, c_, h_, w_ = x.shape
    k_, _, r_, s_ = w.shape
    p_, q_ = h_ + 2 * py - r_ + 1, w_ + 2 * px - s_ + 1
    y = np.zeros((n_, k_, p_, q_))
    for n in range(n_):
        for k in range(k_):
            g = k // GROUP_WIDTH
            for p in range(p_):
                for q in range(q_):
                    acc = 0.0 if bias32 is None else float(bias32[k])
                    for c in range(GROUP_WIDTH):
                        for r in range(r_):
                            ih = p + r - py
                            if ih < 0 or ih >= h_:
                                continue
                            for s in range(s_):
                                iw = q + s - px
                                if 0 <= iw < w_:
                                    acc += x[n, GROUP_WIDTH * g + c, ih, iw] * w[k, c, r, s]
                    y[n, k, p, q] = acc
    return torch.from_numpy(y).float()


def dgrad_loops(dy16, w16, h_, w_, py, px):
    dy, w = _np(dy16), _np(w16)
    n_, k_, p_, q_ = dy.shape
    _, _, r_, s_ = w.shape
    dx = np.zeros((n_, k_, h_, w_))
    for n in range(n_):
        for g in range(k_ // GROUP_WIDTH):
            for c in range(GROUP_WIDTH):
                for h in range(h_):
                    for ww in range(w_):
                        acc = 0.0
                        for j in range(GROUP_WIDTH):
                            for r in range(r_):
                                p = h - r + py
                                if p < 0 or p >= p_:
                                    continue
                                for s in range(s_):
                                    q = ww - s + px
                                    if 0 <= q < q_:
                                        acc += dy[n, GROUP_WIDTH * g + j, p, q] * w[GROUP_WIDTH * g + j, c, r, s]
                        dx[n, GROUP_WIDTH * g + c, h, ww] = acc
    return torch.from_numpy(dx).float()


def wgrad_loops(x16, dy16, r_, s_, py, px):
    x, dy = _np(x16), _np(dy16)
    n_, c_, h_, w_ = x.shape
    _, k_, p_, q_ = dy.shape
    dw = np.zeros((k_, GROUP_WIDTH, r_, s_))
    for k in range(k_):
        g = k // GROUP_WIDTH
        for c in range(GROUP_WIDTH):
            for r in range(r_):
                for s in range(s_):
                    acc = 0.0
                    for n in range(n_):
                        for p in range(p_):
                            ih = p + r - py
                            if ih < 0 or ih >= h_:
                                continue
                            for q in range(q_):
                                iw = q + s - px
                                if 0 <= iw < w_:
                                    acc += x[n, GROUP_WIDTH * g + c, ih, iw] * dy[n, k, p, q]
                    dw[k, c, r, s] = acc
    return torch.from_numpy(dw).float()


# ----------------------------------------------------------------------------
# seeded synthetic arguments
# ----------------------------------------------------------------------------
def make_args(n, c, h, w, r, s, py, px, has_bias=False, seed=0, clip=3.0, weight_init="kaiming"):
    """CPU tensors for one problem: x, w (fp16, channels_last), bias (fp32 or None), dy (fp16).

    Activations are N(0,1) clipped to +-`clip` like the reference's test inputs
    (spio/reflection/arg_info.py:81-85); weights are kaiming-uniform on
    [C,8,R,S] (the nn.Conv2d default) or N(0,1) clipped.
    """
    gen = torch.Generator().manual_seed(seed)
    cl = torch.channels_last
    x = torch.randn(n, c, h, w, generator=gen).clamp_(-clip, clip).half().contiguous(memory_format=cl)
    if weight_init == "kaiming":
        fan_in = GROUP_WIDTH * r * s
        bound = (6.0 / ((1 + 5.0) * fan_in)) ** 0.5  # kaiming_uniform_(a=sqrt(5))
        wt = (torch.rand(c, GROUP_WIDTH, r, s, generator=gen) * 2 - 1) * bound
    else:
        wt = torch.randn(c, GROUP_WIDTH, r, s, generator=gen).clamp_(-clip, clip)
    wt = wt.half().contiguous(memory_format=cl)
    bias = torch.randn(c, generator=gen).float() if has_bias else None
    p, q = h + 2 * py - r + 1, w + 2 * px - s + 1
    dy = torch.randn(n, c, p, q, generator=gen).clamp_(-clip, clip).half().contiguous(memory_format=cl)
    return x, wt, bias, dy


def check_close(actual, expected, acc_depth=None, rtol=NORTH_STAR_RTOL, atol=NORTH_STAR_ATOL, what=""):
    """Elementwise |a-e| <= atol + rtol*|e|; returns the worst ratio for reporting.

    With `acc_depth` the reference's tighter rule is applied instead
    (spio/util/close.py:6-35): rtol 1e-3, atol = depth * 1.6^2 * 1.19e-7 * 3.5.
    """
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} != {tuple(e.shape)}"
    if acc_depth is not None:
        atol = acc_depth * 1.6 * 1.6 * 1.19e-7 * 3.5
        rtol = 1e-3
    err = (a - e).abs()
    tol = atol + rtol * e.abs()
    ok = err <= tol
    if not bool(ok.all()):
        bad = torch.nonzero(~ok)
        i = tuple(int(v) for v in bad[0])
        raise AssertionError(
            f"{what}: {int((~ok).sum())}/{ok.numel()} elements out of tolerance (atol={atol:g}, "
            f"rtol={rtol:g}); first at {i}: actual {float(a[i])} expected {float(e[i])}; "
            f"max |diff| {float(err.max())}"
        )
    return float((err / tol).max())
