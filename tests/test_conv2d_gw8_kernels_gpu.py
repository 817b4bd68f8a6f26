"""GPU parity of the fprop / dgrad / wgrad kernels against the CPU oracle.

Mirrors the kernel-level tests of the reference (tests/test_conv2d_gw8.py:
110-201): sanity shapes, the regression shapes, and seeded samples of the full
shape list, each over several tile configurations, outputs pre-filled with a
sentinel.
"""

import pytest

from helpers import run_bgrad_kernel_test, run_grad_kernel_test, run_kernel_test, sample_params
from spio_amd.kernels import (
    Conv2dGw8BgradConfig,
    Conv2dGw8Config,
    Conv2dGw8Params,
    Conv2dGw8WgradConfig,
    bgrad_is_supported,
    conv2d_gw8_bgrad_kernel_factory,
    conv2d_gw8_kernel_factory,
    conv2d_gw8_wgrad_kernel_factory,
)

pytestmark = pytest.mark.gpu

SANITY = [
    Conv2dGw8Params(n=4, c=64, h=16, w=32, padding=1, r=3, s=3, has_bias=True),
    Conv2dGw8Params(n=4, c=48, h=32, w=32, padding=1, r=3, s=3, has_bias=False),
    Conv2dGw8Params(n=1, c=64, h=8, w=16, padding=1, r=3, s=3, has_bias=False),
    Conv2dGw8Params(n=4, c=128, h=32, w=32, padding=(2, 0), r=4, s=1, has_bias=True),
    Conv2dGw8Params(n=1, c=128, h=64, w=64, padding=7, has_bias=False),
    Conv2dGw8Params(n=6, c=128, h=6, w=5, has_bias=True),
    Conv2dGw8Params(n=3, c=24, h=20, w=19, padding=0, has_bias=False),
    Conv2dGw8Params(n=2, c=40, h=9, w=9, r=5, s=5, padding=2, has_bias=True),
    Conv2dGw8Params(n=2, c=32, h=14, w=14, r=7, s=7, padding=3, has_bias=False),
    Conv2dGw8Params(n=5, c=8, h=7, w=7, r=2, s=5, padding=(1, 2), has_bias=True),
    # one filter row with a bias and an odd row count: the fused bias sum needs its extra step
    Conv2dGw8Params(n=3, c=16, h=9, w=11, r=1, s=3, padding=(0, 1), has_bias=True),
    # one filter row, bias, many rows per image: the bias sum reads a row pair while the next row
    # is staged, which needs a deeper grad_output ring than the one-row weight gradient itself
    Conv2dGw8Params(n=1, c=128, h=32, w=32, r=1, s=1, padding=0, has_bias=True),
    Conv2dGw8Params(n=1, c=128, h=32, w=32, r=1, s=4, padding=(0, 2), has_bias=True),
    # output taller than the input, with a bias: grad_output rows whose x row is all padding
    Conv2dGw8Params(n=2, c=16, h=6, w=6, r=3, s=3, padding=2, has_bias=True),
]


@pytest.mark.parametrize("params", SANITY, ids=lambda p: p.encode())
def test_fprop_sanity(params):
    run_kernel_test(conv2d_gw8_kernel_factory, params)


@pytest.mark.parametrize("params", SANITY, ids=lambda p: p.encode())
def test_dgrad_sanity(params):
    run_grad_kernel_test(conv2d_gw8_kernel_factory, params, igrad=True)


@pytest.mark.parametrize("params", SANITY, ids=lambda p: p.encode())
def test_wgrad_sanity(params):
    run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params)


def test_two_tile_heights_and_prefetch_ramp():
    """Row blocks of two alternating heights (the second half of the grid takes the second height)
    and the ramped prefetch, forward and data gradient: image heights that are and are not
    multiples of the pair, a last pair that lies partly outside the image, images side by side,
    split tiles, a bias, a 5x5 filter, padding that changes the image size."""
    C = Conv2dGw8Config
    cases = [
        (Conv2dGw8Params(n=5, c=64, h=28, w=28, padding=1, has_bias=True),
         [C(groups=8, block_p=9, block_p2=5, prefetch=4), C(groups=4, block_p=18, block_p2=10, prefetch=12, prefetch_start=3, prefetch_rate=2),
          C(groups=8, block_p=5, block_p2=9, prefetch=8, block_n=2, split=2, prefetch_start=2, prefetch_rate=3)]),
        (Conv2dGw8Params(n=3, c=24, h=19, w=20, padding=0, has_bias=False),
         [C(groups=3, block_p=7, block_p2=4, prefetch=4), C(groups=3, block_p=4, block_p2=1, prefetch=2, xcd_chunk=0),
          C(groups=3, block_p=16, block_p2=1, prefetch=4, prefetch_start=2, prefetch_rate=1)]),
        (Conv2dGw8Params(n=2, c=40, h=9, w=9, r=5, s=5, padding=2, has_bias=True),
         [C(groups=5, block_p=3, block_p2=2, prefetch=2), C(groups=5, block_p=6, block_p2=3, prefetch=4, prefetch_start=2, prefetch_rate=2)]),
        (Conv2dGw8Params(n=1, c=128, h=64, w=64, padding=7, has_bias=False),
         [C(groups=8, block_p=20, block_p2=12, prefetch=8, prefetch_start=4, prefetch_rate=2)]),
        (Conv2dGw8Params(n=4, c=128, h=32, w=32, padding=(2, 0), r=4, s=1, has_bias=True),
         [C(groups=8, block_p=10, block_p2=7, prefetch=4)]),
    ]  # fmt: skip
    for params, configs in cases:
        run_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs)
        run_grad_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs, igrad=True)


def test_column_blocks():
    """Workgroups that own a block of output columns (block_q) and stage block_q + S - 1 source
    columns: widths that are and are not multiples of the block, blocks wider than what is left
    at the right edge, 5x5 and even filters (column halo of 4 and 3), padding 0 and padding
    larger than the halo, together with two tile heights; forward and data gradient."""
    C = Conv2dGw8Config
    cases = [
        (Conv2dGw8Params(n=3, c=24, h=9, w=150, padding=1, has_bias=True),
         [C(groups=3, block_p=4, block_q=64, prefetch=4), C(groups=3, block_p=9, block_q=32, prefetch=2, split=2),
          C(groups=3, block_p=3, block_p2=1, block_q=128, prefetch=4)]),
        (Conv2dGw8Params(n=2, c=16, h=7, w=100, r=5, s=5, padding=2, has_bias=False),
         [C(groups=2, block_p=7, block_q=64, prefetch=4), C(groups=2, block_p=2, block_q=16, prefetch=2)]),
        (Conv2dGw8Params(n=2, c=16, h=6, w=77, r=2, s=4, padding=(0, 3), has_bias=True),
         [C(groups=2, block_p=3, block_q=32, prefetch=2), C(groups=1, block_p=5, block_q=48, prefetch=4)]),
        (Conv2dGw8Params(n=2, c=32, h=10, w=70, padding=0, has_bias=False),
         [C(groups=4, block_p=4, block_q=32, prefetch=4)]),
        (Conv2dGw8Params(n=4, c=32, h=64, w=512, padding=1, has_bias=False),
         [C(groups=4, block_p=8, block_q=64, prefetch=8, split=2), C(groups=4, block_p=16, block_q=128, prefetch=4)]),
        (Conv2dGw8Params(n=2, c=64, h=20, w=1024, padding=1, has_bias=True),
         [C(groups=8, block_p=10, block_q=128, prefetch=8), C(groups=4, block_p=7, block_q=256, prefetch=4, split=2)]),
    ]  # fmt: skip
    for params, configs in cases:
        run_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs)
        run_grad_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs, igrad=True)


def test_column_blocks_weight_gradient_and_fused_backward():
    """Column blocks in the weight-gradient kernel (atomics and two-stage) and in the fused
    backward kernel (blocks of 32k columns): each grad_output column is counted by exactly one
    workgroup, the x columns opposite a block's edges come from the neighbouring blocks."""
    W = Conv2dGw8WgradConfig
    B = Conv2dGw8BgradConfig
    cases = [
        (Conv2dGw8Params(n=3, c=24, h=9, w=150, padding=1, has_bias=True),
         [W(groups=3, block_h=4, block_q=64, prefetch=2), W(groups=3, block_h=9, block_q=64, prefetch=2, split=2, two_stage=1),
          W(groups=3, block_h=8, block_q=48, prefetch=2, rows=2)],
         [B(groups=3, block_h=0, block_q=64, prefetch=2), B(groups=3, block_h=7, block_q=64, prefetch=4, split=2), B(groups=3, block_h=4, block_q=32, prefetch=2)]),
        (Conv2dGw8Params(n=2, c=16, h=7, w=100, r=5, s=5, padding=2, has_bias=False),
         [W(groups=2, block_h=7, block_q=64, prefetch=2), W(groups=2, block_h=4, block_q=16, prefetch=2, two_stage=1)],
         [B(groups=2, block_h=0, block_q=32, prefetch=2), B(groups=2, block_h=3, block_q=64, prefetch=2, split=2)]),
        (Conv2dGw8Params(n=2, c=16, h=6, w=77, r=2, s=4, padding=(0, 3), has_bias=True),
         [W(groups=2, block_h=4, block_q=32, prefetch=2)],
         [B(groups=2, block_h=0, block_q=32, prefetch=2)]),
        (Conv2dGw8Params(n=2, c=32, h=10, w=70, padding=0, has_bias=False),
         [W(groups=4, block_h=4, block_q=32, prefetch=2)],
         [B(groups=4, block_h=7, block_q=32, prefetch=2)]),
        (Conv2dGw8Params(n=4, c=32, h=64, w=512, padding=1, has_bias=False),
         [W(groups=4, block_h=8, block_q=64, prefetch=4), W(groups=4, block_h=16, block_q=128, prefetch=2, two_stage=1)],
         [B(groups=4, block_h=14, block_q=64, prefetch=4), B(groups=4, block_h=0, block_q=128, prefetch=2, block_n_iters=2, split=2)]),
        (Conv2dGw8Params(n=2, c=64, h=20, w=1024, padding=1, has_bias=True),
         [W(groups=8, block_h=7, block_q=128, prefetch=2), W(groups=4, block_h=20, block_q=256, prefetch=2, split=2)],
         [B(groups=8, block_h=7, block_q=64, prefetch=2), B(groups=4, block_h=0, block_q=128, prefetch=2, split=2)]),
    ]  # fmt: skip
    for params, wconfigs, bconfigs in cases:
        run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params, configs=wconfigs)
        run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, configs=bconfigs)


def test_weight_gradient_packed_images_skipped_padding_and_pipeline():
    """Small images under large filters: images sharing their halo columns, chunks that hold their
    own images (14x14 under 7x7: two per 32-pixel chunk; 10 wide under 3x3: three), whole-image
    workgroups that skip the steps whose x rows are padding (odd and even first step, one and two
    rows per step; not with a bias), and the pipelined step (MFMAs one step behind the reads) with
    atomics, two stages, split groups, ragged batches and ragged channel blocks."""
    W = Conv2dGw8WgradConfig
    cases = [
        (Conv2dGw8Params(n=10, c=32, h=14, w=14, r=7, s=7, padding=3, has_bias=False),
         [W(groups=4, block_h=14, block_n=4, block_n_iters=2, prefetch=4, two_stage=1),
          W(groups=4, block_h=14, block_n=4, block_n_iters=2, prefetch=4, two_stage=1, pipe=1),
          W(groups=4, block_h=14, block_n=8, prefetch=2, pipe=1),
          W(groups=4, block_h=14, block_n=6, prefetch=2, two_stage=1, split=3, pipe=1),
          W(groups=2, block_h=14, block_n=4, prefetch=2, rows=2, pipe=1),
          W(groups=4, block_h=14, block_n=4, prefetch=2, rows=2, two_stage=1),
          W(groups=4, block_h=7, block_n=4, prefetch=2, pipe=1)]),
        (Conv2dGw8Params(n=7, c=24, h=14, w=14, r=7, s=7, padding=3, has_bias=True),
         [W(groups=3, block_h=14, block_n=4, prefetch=2, pipe=1), W(groups=2, block_h=14, block_n=4, prefetch=4, two_stage=1)]),
        (Conv2dGw8Params(n=13, c=16, h=9, w=10, padding=1, has_bias=False),
         [W(groups=2, block_h=9, block_n=6, prefetch=2), W(groups=2, block_h=9, block_n=6, prefetch=2, pipe=1),
          W(groups=2, block_h=9, block_n=3, block_n_iters=2, prefetch=4, pipe=1, two_stage=1)]),
        (Conv2dGw8Params(n=9, c=16, h=12, w=15, r=5, s=5, padding=2, has_bias=False),
         [W(groups=2, block_h=12, block_n=4, prefetch=2, pipe=1), W(groups=2, block_h=12, block_n=4, prefetch=2, rows=2, pipe=1),
          W(groups=2, block_h=12, block_n=2, prefetch=4)]),
        (Conv2dGw8Params(n=5, c=16, h=11, w=13, r=4, s=6, padding=(1, 4), has_bias=False),
         [W(groups=2, block_h=9, block_n=4, prefetch=2, pipe=1), W(groups=2, block_h=9, block_n=2, prefetch=2)]),
        (Conv2dGw8Params(n=6, c=64, h=56, w=56, padding=1, has_bias=False),
         [W(groups=4, block_h=56, prefetch=2, rows=2, pipe=1), W(groups=8, block_h=56, prefetch=4, pipe=1, block_n_iters=2)]),
        (Conv2dGw8Params(n=16, c=48, h=7, w=7, padding=1, has_bias=True),
         [W(groups=6, block_h=7, block_n=8, prefetch=2, pipe=1), W(groups=6, block_h=7, block_n=4, block_n_iters=2, prefetch=2)]),
    ]  # fmt: skip
    for params, configs in cases:
        run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params, configs=configs)


# shapes the fused backward kernel has a configuration for: any padding, odd and even filter
# sizes (7x7 needs more registers than a wave has and stays with the separate kernels)
FUSED = [p for p in SANITY if bgrad_is_supported(p) and list(conv2d_gw8_bgrad_kernel_factory.configs(p))] + [
    Conv2dGw8Params(n=5, c=24, h=7, w=9, r=1, s=1, padding=0, has_bias=True),
    Conv2dGw8Params(n=3, c=16, h=10, w=12, r=5, s=3, padding=(2, 1), has_bias=False),
    Conv2dGw8Params(n=3, c=72, h=19, w=40, padding=1, has_bias=True),
    # output narrower and taller than the input, and the other way round
    Conv2dGw8Params(n=3, c=16, h=13, w=18, r=5, s=3, padding=(3, 0), has_bias=True),
    Conv2dGw8Params(n=3, c=16, h=13, w=18, r=3, s=5, padding=(0, 4), has_bias=False),
]


@pytest.mark.parametrize("params", FUSED, ids=lambda p: p.encode())
def test_bgrad_sanity(params):
    """Fused data + weight (+ bias) gradient kernel, first configurations of every shape."""
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params)


def test_bgrad_two_stage():
    """Fused backward kernel with two-stage publishing: blocks of partial sums and the second
    kernel that stores their sum.  Channel blocks with missing groups, row and column blocks,
    images side by side, image blocks per workgroup, split groups, with and without a bias."""
    C = Conv2dGw8BgradConfig
    cases = [
        (Conv2dGw8Params(n=5, c=24, h=20, w=28, padding=1, has_bias=True),
         [C(groups=2, block_h=7, block_n=2, block_n_iters=1, prefetch=2, two_stage=1),
          C(groups=3, block_h=0, block_n=2, block_n_iters=2, prefetch=4, split=2, two_stage=1)]),
        (Conv2dGw8Params(n=3, c=72, h=19, w=40, padding=1, has_bias=False),
         [C(groups=4, block_h=7, block_n=1, block_n_iters=1, prefetch=2, two_stage=1),
          C(groups=9, block_h=14, block_n=1, block_n_iters=2, prefetch=2, two_stage=1)]),
        (Conv2dGw8Params(n=2, c=40, h=9, w=9, r=5, s=5, padding=2, has_bias=True),
         [C(groups=5, block_h=0, block_n=2, prefetch=2, two_stage=1)]),
        (Conv2dGw8Params(n=3, c=24, h=9, w=150, padding=1, has_bias=True),
         [C(groups=3, block_h=4, block_q=64, prefetch=2, two_stage=1)]),
        (Conv2dGw8Params(n=5, c=32, h=17, w=21, r=4, s=4, padding=(0, 3), has_bias=True),
         [C(groups=4, block_h=5, block_n=1, block_n_iters=1, prefetch=2, two_stage=1)]),
    ]  # fmt: skip
    for params, configs in cases:
        run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, configs=configs)


def test_bgrad_when_the_image_size_changes():
    """Paddings other than (R-1)/2, and even filter sizes: the kernel works on a domain that holds
    both tensors at offsets that reproduce the padding.  Row blocks that lie partly or wholly
    outside the smaller tensor, images side by side, split groups, a bias; the reference's sampled
    shapes draw their padding from the same range (tests/test_conv2d_gw8.py:80-85) and its
    regression cases hold r=4, s=1, padding=(2, 0) (tests/test_conv2d_gw8.py:176-180)."""
    C = Conv2dGw8BgradConfig
    # output smaller than the input
    params = Conv2dGw8Params(n=5, c=48, h=20, w=28, padding=0, has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_n=2, block_n_iters=1, prefetch=2, split=2),
                                   C(groups=6, block_h=7, block_n=1, block_n_iters=2, prefetch=4, split=1),
                                   C(groups=4, block_h=1, block_n=2, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip
    # smaller in one direction, larger in the other
    params = Conv2dGw8Params(n=5, c=48, h=20, w=28, padding=(0, 3), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_n=2, block_n_iters=1, prefetch=2, split=2),
                                   C(groups=6, block_h=7, block_n=1, block_n_iters=2, prefetch=4, split=1)])  # fmt: skip
    # output taller than the input: whole row blocks of grad_output face only padding rows of x
    params = Conv2dGw8Params(n=5, c=48, h=20, w=28, padding=(3, 0), has_bias=False)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_n=2, block_n_iters=2, prefetch=4, split=1),
                                   C(groups=6, block_h=7, block_n=1, block_n_iters=2, prefetch=4, split=1),
                                   C(groups=4, block_h=2, block_n=1, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip
    # 5x5 filter
    params = Conv2dGw8Params(n=3, c=16, h=13, w=18, r=5, s=5, padding=(0, 4), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=2, block_h=5, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   C(groups=2, block_h=3, block_n=2, block_n_iters=1, prefetch=2, split=2)])  # fmt: skip
    # even filter sizes: the output is one row or column larger or smaller than the input
    params = Conv2dGw8Params(n=4, c=128, h=32, w=32, r=4, s=1, padding=(2, 0), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=8, block_h=7, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   C(groups=4, block_h=0, block_n=2, block_n_iters=2, prefetch=4, split=1)])  # fmt: skip
    params = Conv2dGw8Params(n=5, c=32, h=17, w=21, r=4, s=4, padding=(0, 3), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_h=5, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   C(groups=2, block_h=0, block_n=2, block_n_iters=2, prefetch=4, split=2),
                                   C(groups=4, block_h=1, block_n=1, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip
    params = Conv2dGw8Params(n=5, c=32, h=17, w=21, r=2, s=2, padding=(1, 0), has_bias=False)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_h=5, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   C(groups=2, block_h=0, block_n=2, block_n_iters=2, prefetch=4, split=2)])  # fmt: skip
    params = Conv2dGw8Params(n=5, c=32, h=17, w=21, r=3, s=2, padding=(1, 1), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=4, block_h=7, block_n=2, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip
    # one filter row, padding rows above and below: the bias sum's extra step
    params = Conv2dGw8Params(n=2, c=16, h=9, w=11, r=1, s=3, padding=(2, 0), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[C(groups=2, block_h=3, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   C(groups=2, block_h=0, block_n=2, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip


def test_bgrad_explicit_configs():
    """Split groups, images side by side, several image blocks per workgroup, a group count
    that does not divide the channel blocks, a batch that does not fill the last block."""
    params = Conv2dGw8Params(n=5, c=48, h=20, w=28, padding=1, has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[Conv2dGw8BgradConfig(groups=4, block_n=2, block_n_iters=1, prefetch=2, split=2),
                                   Conv2dGw8BgradConfig(groups=4, block_n=2, block_n_iters=2, prefetch=4, split=1),
                                   Conv2dGw8BgradConfig(groups=6, block_n=2, block_n_iters=1, prefetch=2, split=2),
                                   Conv2dGw8BgradConfig(groups=4, block_n=4, block_n_iters=1, prefetch=2, split=2),
                                   # row blocks with halo rows, a last block that is not full (20 = 7+7+6)
                                   Conv2dGw8BgradConfig(groups=4, block_h=7, block_n=2, block_n_iters=1, prefetch=2, split=1),
                                   Conv2dGw8BgradConfig(groups=6, block_h=14, block_n=1, block_n_iters=2, prefetch=4, split=1),
                                   Conv2dGw8BgradConfig(groups=4, block_h=1, block_n=2, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip
    # 5x5 filter (two halo rows), odd block height, bias
    params = Conv2dGw8Params(n=3, c=16, h=13, w=18, r=5, s=5, padding=2, has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[Conv2dGw8BgradConfig(groups=2, block_h=5, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   Conv2dGw8BgradConfig(groups=2, block_h=3, block_n=2, block_n_iters=1, prefetch=2, split=2)])  # fmt: skip
    # one filter row (no halo rows) with a bias: the bias sum's extra step, odd block height
    params = Conv2dGw8Params(n=2, c=16, h=9, w=11, r=1, s=3, padding=(0, 1), has_bias=True)
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[Conv2dGw8BgradConfig(groups=2, block_h=3, block_n=1, block_n_iters=1, prefetch=2, split=1),
                                   Conv2dGw8BgradConfig(groups=2, block_h=4, block_n=1, block_n_iters=1, prefetch=2, split=1)])  # fmt: skip


def test_odd_image_counts_on_small_images():
    """7x7 images: 3 and 7 images side by side fill the 32-pixel chunks of the weight gradient's
    contraction better than powers of two; a batch that leaves the last block ragged."""
    from spio_amd.kernels import Conv2dGw8WgradConfig

    params = Conv2dGw8Params(n=17, c=64, h=7, w=7, padding=1, has_bias=True)
    run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params,
                         configs=[Conv2dGw8WgradConfig(groups=4, block_h=7, block_n=7, block_n_iters=1, prefetch=4),
                                  Conv2dGw8WgradConfig(groups=8, block_h=7, block_n=7, block_n_iters=2, prefetch=2, rows=2),
                                  Conv2dGw8WgradConfig(groups=4, block_h=4, block_n=3, block_n_iters=2, prefetch=2, two_stage=1)])  # fmt: skip
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params,
                          configs=[Conv2dGw8BgradConfig(groups=8, block_h=0, block_n=7, block_n_iters=1, prefetch=2, split=1),
                                   Conv2dGw8BgradConfig(groups=4, block_h=0, block_n=3, block_n_iters=2, prefetch=4, split=1)])  # fmt: skip


def test_bgrad_is_offered_for_every_padding_and_filter_parity():
    for params in (Conv2dGw8Params(n=1, c=8, h=8, w=8, padding=0), Conv2dGw8Params(n=1, c=8, h=8, w=8, padding=2),
                   Conv2dGw8Params(n=1, c=8, h=8, w=8, r=4, s=1, padding=(2, 0)),
                   Conv2dGw8Params(n=1, c=8, h=8, w=8, r=2, s=5, padding=(1, 2))):  # fmt: skip
        assert bgrad_is_supported(params) and list(conv2d_gw8_bgrad_kernel_factory.configs(params))
    # 7x7: no configuration fits the registers
    assert list(conv2d_gw8_bgrad_kernel_factory.configs(Conv2dGw8Params(n=2, c=32, h=14, w=14, r=7, s=7, padding=3))) == []


def test_fprop_explicit_configs():
    """Explicit tile configurations, like the reference's regression cases
    (tests/test_conv2d_gw8.py:117-142): a group count that does not divide the
    channel blocks evenly and a one-image tile."""
    params = Conv2dGw8Params(n=4, c=48, h=32, w=32, padding=1)
    run_kernel_test(conv2d_gw8_kernel_factory, params,
                    configs=[Conv2dGw8Config(groups=4, block_p=8, block_n=2, split=1),
                             Conv2dGw8Config(groups=6, block_p=7, block_n=1, split=2)])  # fmt: skip
    params = Conv2dGw8Params(n=1, c=64, h=8, w=16, padding=1)
    run_kernel_test(conv2d_gw8_kernel_factory, params,
                    configs=[Conv2dGw8Config(groups=8, block_p=8, block_n=1)])  # fmt: skip


def _image(groups, block_n, split, iters, buffers=2, movers=0):
    return Conv2dGw8Config(groups=groups, block_p=0, block_n=block_n, split=split, prefetch=buffers,
                           variant="image", block_n_iters=iters, halo_cached=0, xcd_chunk=0,
                           movers=movers)  # fmt: skip


def _movers(groups, block_n, split, iters, movers=4):
    return _image(groups, block_n, split, iters, 2, movers)


IMAGE_CASES = [
    # 7x7 filter on 14x14: accumulators split over 1, 2, 4 waves; 1..4 image blocks per workgroup;
    # a batch that does not fill the last workgroup's blocks
    (Conv2dGw8Params(n=7, c=64, h=14, w=14, r=7, s=7, padding=3),
     [_image(8, 1, 1, 1), _image(8, 1, 1, 5), _image(4, 1, 4, 2), _image(4, 1, 2, 3, 1), _image(4, 1, 2, 16),
      _image(8, 1, 1, 2, 1), _image(4, 2, 2, 3, 1),
      # data-mover waves: 1..5 blocks per workgroup, split accumulators, two mover waves
      _movers(8, 1, 1, 1), _movers(8, 1, 1, 4), _movers(4, 1, 2, 5), _movers(4, 1, 1, 2, movers=2), _movers(2, 2, 2, 3)]),
    # 3x3 with a bias, images side by side, a group count that leaves idle waves (5 groups, 4 per block)
    (Conv2dGw8Params(n=9, c=40, h=14, w=14, has_bias=True),
     [_image(4, 2, 1, 2), _image(4, 1, 2, 1, 1), _image(5, 1, 1, 4), _image(2, 4, 2, 1), _image(5, 2, 1, 3, 1),
      _movers(4, 2, 1, 2), _movers(5, 1, 1, 4, movers=5), _movers(2, 4, 2, 1)]),
    # 7x7 images
    (Conv2dGw8Params(n=12, c=64, h=7, w=7, has_bias=True), [_image(8, 2, 1, 2), _image(8, 2, 2, 1), _image(4, 4, 1, 3), _image(8, 4, 1, 3, 1),
      _movers(8, 2, 1, 2), _movers(4, 4, 1, 3)]),
    # 5x5 (three accumulators: splits 1 and 3), non-square image
    (Conv2dGw8Params(n=5, c=32, h=9, w=12, r=5, s=5, padding=2, has_bias=True), [_image(4, 1, 3, 2), _image(4, 2, 1, 2, 1), _movers(4, 1, 3, 2)]),
    # asymmetric filter and padding, output larger than the input (the data gradient then crops)
    (Conv2dGw8Params(n=3, c=16, h=6, w=8, r=3, s=3, padding=2), [_image(2, 1, 1, 2), _image(2, 2, 2, 1), _image(2, 1, 1, 3, 1), _movers(2, 1, 1, 3)]),
    (Conv2dGw8Params(n=4, c=16, h=10, w=6, r=4, s=1, padding=(2, 0), has_bias=True), [_image(2, 2, 2, 2), _movers(2, 2, 2, 2)]),
    (Conv2dGw8Params(n=2, c=16, h=8, w=8, r=3, s=3, padding=0), [_image(2, 1, 1, 2)]),
]


@pytest.mark.parametrize("params,configs", IMAGE_CASES, ids=lambda v: v.encode() if hasattr(v, "encode") else "")
def test_whole_image_kernel_configs(params, configs):
    """The whole-image forward / data-gradient kernel over explicit configurations."""
    run_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs)
    run_grad_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs, igrad=True)


def test_stores_keep_their_data_registers():
    """Configurations whose compiled code once wrote a result into the first data register of a
    16-byte buffer store in the instruction behind it (row offset in a scalar register: no wait
    state is inserted for that form), which now and then stored stray values in the first two
    channels of some pixels of one output row.  Three runs each, full-size grids."""
    params = Conv2dGw8Params(n=256, c=256, h=14, w=14, r=7, s=7, padding=3)
    for seed in range(3):
        run_kernel_test(conv2d_gw8_kernel_factory, params, seed=seed,
                        configs=[Conv2dGw8Config(groups=4, block_p=14, block_n=2, prefetch=8),
                                 Conv2dGw8Config(groups=4, block_p=14, block_n=2, prefetch=4)])  # fmt: skip
    params = Conv2dGw8Params(n=8, c=64, h=56, w=56)
    for seed in range(3):
        run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, seed=seed,
                              configs=[Conv2dGw8BgradConfig(groups=8, block_h=0, prefetch=2, split=2)])  # fmt: skip


@pytest.mark.slow
@pytest.mark.parametrize("params", sample_params(seed=1), ids=lambda p: p.encode())
def test_fprop_sampled(params):
    run_kernel_test(conv2d_gw8_kernel_factory, params)


@pytest.mark.slow
@pytest.mark.parametrize("params", sample_params(seed=2), ids=lambda p: p.encode())
def test_dgrad_sampled(params):
    run_grad_kernel_test(conv2d_gw8_kernel_factory, params, igrad=True)


@pytest.mark.slow
@pytest.mark.parametrize("params", sample_params(seed=3), ids=lambda p: p.encode())
def test_wgrad_sampled(params):
    run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params)


def _sampled_fused(seed, count=6):
    """Seeded draw from the reference's model-derived shapes the fused backward kernel supports."""
    import random

    from helpers import reference_test_params

    pool = [p for p in reference_test_params(True) + reference_test_params(False)
            if bgrad_is_supported(p) and list(conv2d_gw8_bgrad_kernel_factory.configs(p))]  # fmt: skip
    return random.Random(seed).sample(pool, min(count, len(pool)))


@pytest.mark.slow
@pytest.mark.parametrize("params", _sampled_fused(seed=4), ids=lambda p: p.encode())
def test_bgrad_sampled(params):
    run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params)
