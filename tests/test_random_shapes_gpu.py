"""GPU parity on seeded random shapes outside the reference's shape list.

The reference's kernel tests draw from a fixed list (tests/test_conv2d_gw8.py:67-107: square
filters up to 5x5, padding r//2 or a few fixed values).  These draws add what that list leaves
out — filters up to 7x7 with r != s, padding between zero and more than half the filter, image
sizes and batches of every parity — and run every kernel family over a seeded spread of its legal
tile configurations.  SPIO_RANDOM_SHAPES sets the number of shapes (default 8, a quarter of a
minute; several hundred take a quarter of an hour), SPIO_RANDOM_SEED the draw.
"""

import os

import pytest

from helpers import pick_configs, random_params, run_bgrad_kernel_test, run_grad_kernel_test, run_kernel_test
from spio_amd.hip import get_device_attributes
from spio_amd.kernels import (
    bgrad_is_supported,
    conv2d_gw8_bgrad_kernel_factory,
    conv2d_gw8_kernel_factory,
    conv2d_gw8_wgrad_kernel_factory,
)

pytestmark = pytest.mark.gpu

COUNT = int(os.environ.get("SPIO_RANDOM_SHAPES", "8"))
SEED = int(os.environ.get("SPIO_RANDOM_SEED", "7"))
CONFIGS = int(os.environ.get("SPIO_RANDOM_CONFIGS", "4"))


@pytest.mark.parametrize("index,params", list(enumerate(random_params(SEED, COUNT))), ids=lambda v: v.encode() if hasattr(v, "encode") else str(v))  # fmt: skip
def test_random_shape_all_families(index, params):
    attr = get_device_attributes(0)
    seed = SEED * 1000 + index

    def spread(factory, **kw):
        return pick_configs(factory, params, attr, None, limit=CONFIGS, seed=seed, **kw)

    run_kernel_test(conv2d_gw8_kernel_factory, params, configs=spread(conv2d_gw8_kernel_factory), seed=index)
    run_grad_kernel_test(conv2d_gw8_kernel_factory, params, igrad=True, seed=index,
                         configs=spread(conv2d_gw8_kernel_factory, igrad=True))  # fmt: skip
    run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params, seed=index,
                         configs=spread(conv2d_gw8_wgrad_kernel_factory))  # fmt: skip
    if bgrad_is_supported(params):
        fused = spread(conv2d_gw8_bgrad_kernel_factory)
        if fused:
            run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, configs=fused, seed=index)
