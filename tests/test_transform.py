"""Model conversion: exactly the eligible convolutions are replaced and share parameters
(reference procedure: spio/src_tests/run_test.py:205-246).  The structural part runs on CPU;
the numerical part needs the GPU."""

import pytest
import torch
from torch import nn

from spio_amd.kernels import Conv2dGw8Params
from spio_amd.layers import Conv2dGw8
from spio_amd.transform import count_replaceable, scan_modules, transform


class Block(nn.Module):
    def __init__(self, c=32):
        super().__init__()
        self.stem = nn.Conv2d(3, c, 3, padding=1)  # not eligible: C_in != C_out
        self.inner = nn.Sequential(nn.Conv2d(c, c, 3, padding=1, groups=c // 8), nn.ReLU())
        self.wide = nn.Conv2d(c, c, 7, padding=3, groups=c // 8)  # kernel size > 5: not matched
        self.dw = nn.Conv2d(c, c, 5, padding=2, groups=c // 8, bias=False)

    def forward(self, x):
        x = self.stem(x)
        x = self.inner(x)
        return self.dw(x) + self.wide(x)


def test_transform_replaces_exactly_the_eligible_modules():
    model = Block()
    assert count_replaceable(model) == 2
    new = transform(model)
    kinds = {name: type(m) for name, m in new.named_modules()}
    assert kinds["inner.0"] is Conv2dGw8 and kinds["dw"] is Conv2dGw8
    assert kinds["stem"] is nn.Conv2d and kinds["wide"] is nn.Conv2d
    assert new.get_submodule("inner.0").weight is model.inner[0].weight  # shared
    assert new.get_submodule("dw").bias is None
    assert count_replaceable(new) == 0


def test_scan_modules_reports_params():
    model = Block()
    found = scan_modules(model, torch.zeros(2, 3, 12, 10))
    assert found == [
        Conv2dGw8Params(n=2, c=32, h=12, w=10, padding=(1, 1), r=3, s=3, has_bias=True),
        Conv2dGw8Params(n=2, c=32, h=12, w=10, padding=(2, 2), r=5, s=5, has_bias=False),
    ]


@pytest.mark.gpu
def test_transformed_model_matches_original():
    """The transformed model on the GPU against the original model in fp32 on the CPU (torch's
    host convolution, the oracle's own reference), not against the GPU library's convolution."""
    import copy

    torch.manual_seed(0)
    cpu_model = Block().float()
    model = copy.deepcopy(cpu_model).cuda().to(memory_format=torch.channels_last)
    new = transform(model)
    x = torch.randn(2, 3, 16, 16)
    with torch.no_grad():
        want = cpu_model(x)
        with torch.autocast(device_type="cuda", dtype=torch.float16):
            got = new(x.cuda().contiguous(memory_format=torch.channels_last))
    # fp16 activations between the layers: a few roundings of O(1) values
    torch.testing.assert_close(got.float().cpu(), want, rtol=1e-2, atol=2e-2)
