"""ConvNeXt-Tiny-shaped network whose 7x7 depthwise convolutions are replaced by 3x3 convolutions
with group width 8 (the fifth benchmark configuration), for the benchmark and the tests.  The
reference ships no such model (its nearest relative is the block in scripts/profile_block.py:75-114).  Stages of widths 96/192/384/768 at 56/28/14/7 spatial for 224x224 inputs,
depths 3/3/9/3, LayerNorm + 4x MLP + GELU, 1000-class head.  Layer scale is initialised to 1 (not
the usual 1e-6) so that the convolutions reach the logits and a wrong convolution shows."""

import torch
from torch import nn


class LayerNorm2d(nn.LayerNorm):
    """LayerNorm over the channel dimension of an NCHW tensor."""

    def forward(self, x):
        return super().forward(x.permute(0, 2, 3, 1)).permute(0, 3, 1, 2)


class Block(nn.Module):
    def __init__(self, dim, make_conv):
        super().__init__()
        self.conv = make_conv(dim)
        self.norm = nn.LayerNorm(dim)
        self.fc1 = nn.Linear(dim, 4 * dim)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(4 * dim, dim)
        self.gamma = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        y = self.conv(x).permute(0, 2, 3, 1)
        y = self.fc2(self.act(self.fc1(self.norm(y)))) * self.gamma
        return x + y.permute(0, 3, 1, 2)


def plain_conv(dim):
    return nn.Conv2d(dim, dim, 3, padding=1, groups=dim // 8)


class ConvNeXtGw8(nn.Module):
    def __init__(self, make_conv=plain_conv, widths=(96, 192, 384, 768), depths=(3, 3, 9, 3), classes=1000,
                 norm2d=LayerNorm2d):
        super().__init__()
        layers = [nn.Conv2d(3, widths[0], 4, stride=4), norm2d(widths[0])]
        for i, (w, d) in enumerate(zip(widths, depths)):
            if i > 0:
                layers += [norm2d(widths[i - 1]), nn.Conv2d(widths[i - 1], w, 2, stride=2)]
            layers += [Block(w, make_conv) for _ in range(d)]
        self.features = nn.Sequential(*layers)
        self.norm = nn.LayerNorm(widths[-1])
        self.head = nn.Linear(widths[-1], classes)

    def forward(self, x):
        x = self.features(x)
        return self.head(self.norm(x.mean(dim=(2, 3))))
