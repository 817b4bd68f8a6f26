"""Tensor comparison with tolerances derived from the accumulation depth.

Reference: spio/util/close.py:6-35 (tolerance rule) and :38-50 (elementwise
test |a - e| <= atol + rtol * |e|).
"""

import torch

FLOAT16_PRECISION = 5e-4
FLOAT32_PRECISION = 1.19e-7


def acc_depth_tolerances(acc_depth, abs_mean=1.6, atol_fudge=3.5, rtol_fudge=2.0):
    """(atol, rtol) for fp16 operands accumulated `acc_depth` deep in fp32."""
    atol = acc_depth * abs_mean * abs_mean * FLOAT32_PRECISION * atol_fudge
    rtol = FLOAT16_PRECISION * rtol_fudge
    return atol, rtol


def assert_all_close_with_acc_depth(
    actual, expected, msg=None, acc_depth=None, abs_mean=1.6, atol_fudge=3.5, rtol_fudge=2.0
):
    """Compare with atol scaled by the number of accumulated products."""
    atol, rtol = acc_depth_tolerances(acc_depth, abs_mean, atol_fudge, rtol_fudge)
    assert_all_close(actual, expected, atol=atol, rtol=rtol, msg=msg)


def assert_all_close(actual, expected, atol=0.0, rtol=0.0, msg=None, max_errors=16):
    """Raise AssertionError listing the first offending elements."""
    assert actual.shape == expected.shape, f"shape {actual.shape} != {expected.shape}"
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    err = (a - e).abs()
    tol = atol + rtol * e.abs()
    bad = ~(err <= tol)  # also catches NaN
    if not bool(bad.any()):
        return
    idx = torch.nonzero(bad)
    lines = [
        f"{int(bad.sum())} of {bad.numel()} elements differ (atol={atol:g}, rtol={rtol:g}); "
        f"max |diff| = {float(err[~torch.isnan(err)].max()) if bool((~torch.isnan(err)).any()) else float('nan'):g}"
    ]
    for i in idx[:max_errors]:
        t = tuple(int(v) for v in i)
        lines.append(
            f"  {list(t)}: actual {float(a[t]):.6f} expected {float(e[t]):.6f} "
            f"|diff| {float(err[t]):.6f} > {float(tol[t]):.6f}"
        )
    if msg:
        lines.append(msg)
    raise AssertionError("\n".join(lines))
