"""ctypes loader of the C oracle -- TEST INFRASTRUCTURE ONLY (see conv2d_gw8_oracle.c)."""

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libconv2d_gw8_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with make/gcc."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libconv2d_gw8_oracle.so"],
                       check=True, capture_output=True)  # fmt: skip
    return LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib


def _u16(t: torch.Tensor) -> np.ndarray:
    """Physical NHWC (or KRSC) fp16 bits of a 4-D channels_last-able tensor."""
    return t.detach().cpu().half().permute(0, 2, 3, 1).contiguous().view(torch.int16).numpy().view(np.uint16)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def fprop_c(x16, w16, bias32, py, px):
    """fp32 NCHW-shaped result of the C forward statement."""
    n, c, h, w = x16.shape
    r, s = w16.shape[2:]
    p, q = h + 2 * py - r + 1, w + 2 * px - s + 1
    xs, ws = _u16(x16), _u16(w16)
    y = np.zeros((n, p, q, c), dtype=np.float32)
    b = None if bias32 is None else np.ascontiguousarray(bias32.detach().cpu().float().numpy())
    _load().gw8_fprop_f32(_ptr(xs), _ptr(ws), None if b is None else _ptr(b), _ptr(y),
                          n, c, h, w, r, s, py, px)  # fmt: skip
    return torch.from_numpy(y).permute(0, 3, 1, 2)


def dgrad_c(dy16, w16, h, w, py, px):
    n, c, _p, _q = dy16.shape
    r, s = w16.shape[2:]
    ds, ws = _u16(dy16), _u16(w16)
    dx = np.zeros((n, h, w, c), dtype=np.float32)
    _load().gw8_dgrad_f32(_ptr(ds), _ptr(ws), _ptr(dx), n, c, h, w, r, s, py, px)
    return torch.from_numpy(dx).permute(0, 3, 1, 2)


def wgrad_c(x16, dy16, r, s, py, px):
    n, c, h, w = x16.shape
    xs, ds = _u16(x16), _u16(dy16)
    dw = np.zeros((c, r, s, 8), dtype=np.float32)
    _load().gw8_wgrad_f32(_ptr(xs), _ptr(ds), _ptr(dw), n, c, h, w, r, s, py, px)
    return torch.from_numpy(dw).permute(0, 3, 1, 2)


def dbias_c(dy16):
    n, c, p, q = dy16.shape
    ds = _u16(dy16)
    db = np.zeros((c,), dtype=np.float32)
    _load().gw8_dbias_f32(_ptr(ds), _ptr(db), n, c, p, q)
    return torch.from_numpy(db)
