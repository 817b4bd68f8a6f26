"""Every shape of the reference's kernel-test lists (spio/src_tests/Conv2dGw8Params.dat and the
parameter grid of tests/test_conv2d_gw8.py: 270 shapes here), every kernel family, against the
CPU oracle: by default the first (best-ranked) configuration of every MFMA kernel (row-streaming
and, where the shape has one, whole-image with and without mover waves) for every shape and one random other configuration for
every third shape (a few minutes on one MI355X); SPIO_EXHAUSTIVE=1 takes five configurations per
kernel family instead (about 15 minutes).
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

pytestmark = [pytest.mark.gpu, pytest.mark.slow]
FULL = os.environ.get("SPIO_EXHAUSTIVE", "0") == "1"

SHAPES = reference_test_params(True) + reference_test_params(False)
CHUNK = 10
CONFIGS_PER_KERNEL = 5


def _pick(factory, params, attr, rng, second=True, **kw):
    every = list(factory.configs(params, attr, **kw))
    rows = [c for c in every if getattr(c, "variant", "mfma") == "mfma"]    # row-streaming kernels
    image = [c for c in every if getattr(c, "variant", "mfma") == "image"]  # whole-image kernel
    movers = [c for c in image if getattr(c, "movers", 0)]                  # ... with data-mover waves
    plain = [c for c in image if not getattr(c, "movers", 0)]
    first = rows[:1] + plain[:1] + movers[:1]
    rest = [c for c in rows + image if c not in first]
    if FULL:
        return first + rng.sample(rest, min(CONFIGS_PER_KERNEL - len(first), len(rest)))
    return first + (rng.sample(rest, 1) if second and rest else [])


@pytest.mark.parametrize("chunk", range((len(SHAPES) + CHUNK - 1) // CHUNK))
def test_all_reference_shapes(chunk):
    from spio_amd.hip import get_device_attributes

    attr = get_device_attributes(0)
    rng = random.Random(int(os.environ.get("SPIO_EXHAUSTIVE_SEED", "1")) * 1000 + chunk)
    for i, params in enumerate(SHAPES[chunk * CHUNK : (chunk + 1) * CHUNK]):
        second = (chunk * CHUNK + i) % 3 == 0
        configs = _pick(conv2d_gw8_kernel_factory, params, attr, rng, second)
        if configs:
            run_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs)
        configs = _pick(conv2d_gw8_kernel_factory, params, attr, rng, second, igrad=True)
        if configs:
            run_grad_kernel_test(conv2d_gw8_kernel_factory, params, configs=configs, igrad=True)
        configs = _pick(conv2d_gw8_wgrad_kernel_factory, params, attr, rng, second)
        if configs:
            run_grad_kernel_test(conv2d_gw8_wgrad_kernel_factory, params, configs=configs)
        configs = _pick(conv2d_gw8_bgrad_kernel_factory, params, attr, rng, second)
        if configs:
            run_bgrad_kernel_test(conv2d_gw8_bgrad_kernel_factory, params, configs=configs)
