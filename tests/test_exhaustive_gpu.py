"""Every shape of the reference's kernel-test lists (spio/src_tests/Conv2dGw8Params.dat and the
parameter grid of tests/test_conv2d_gw8.py: 270 shapes here), every kernel family, several
random tile configurations each, against the CPU oracle.  About 15 minutes on one MI355X, so it
only runs when SPIO_EXHAUSTIVE=1; the default suite draws seeded samples from the same lists.
"""

import os
import random

import pytest

from helpers import (
    reference_test_params,
    run_bgrad_kernel_test,
    run_grad_kernel_test,
    run_kernel_test,
)
from spio_amd.kernels import (
    conv2d_gw8_bgrad_kernel_factory,
    conv2d_gw8_kernel_factory,
    conv2d_gw8_wgrad_kernel_factory,
)

pytestmark = [
    pytest.mark.gpu,
    pytest.mark.slow,
    pytest.mark.skipif(os.environ.get("SPIO_EXHAUSTIVE", "0") != "1", reason="set SPIO_EXHAUSTIVE=1 to run"),
]

SHAPES = reference_test_params(True) + reference_test_params(False)
CHUNK = 10
CONFIGS_PER_KERNEL = 5


def _pick(factory, params, attr, rng, **kw):
    configs = [c for c in factory.configs(params, attr, **kw) if getattr(c, "variant", "mfma") == "mfma"]
    return rng.sample(configs, min(CONFIGS_PER_KERNEL, len(configs)))


@pytest.mark.parametrize("chunk", range((len(SHAPES) + CHUNK - 1) // CHUNK))
def test_all_reference_shapes(chunk):
    from spio_amd.hip import get_device_attributes

    attr = get_device_attributes(0)
    rng = random.Random(int(os.environ.get("SPIO_EXHAUSTIVE_SEED", "1")) * 1000 + chunk)
    for params in SHAPES[chunk * CHUNK : (chunk + 1) * CHUNK]:
        configs = _pick(conv2d_gw8_kernel_factory, params, attr, rng)
        if configs:
            run_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs)
        configs = _pick(conv2d_gw8_kernel_factory, params, attr, rng, igrad=True)
        if configs:
            run_grad_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs, igrad=True)
        configs = _pick(conv2d_gw8_wgrad_kernel_factory, params, attr, rng)
        if configs:
            run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params, configs=configs)
        configs = _pick(conv2d_gw8_bgrad_kernel_factory, params, attr, rng)
        if configs:
            run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, configs=configs)
