"""Memory-format conversion (reference: spio/util/tensor_format.py:8-17)."""

import torch


def to_channels_last(*args):
    """Return args with every 4-D tensor made channels_last contiguous.

    A tensor that already has channels_last strides is returned as is (no
    copy); anything else (None, 1-D bias) passes through untouched.
    """
    out = []
    for t in args:
        if isinstance(t, torch.Tensor) and t.dim() == 4:
            t = t.contiguous(memory_format=torch.channels_last)
        out.append(t)
    return tuple(out)
