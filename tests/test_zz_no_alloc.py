"""spio_hip_launch_scratch: the two-stage weight gradient with the library's static device
workspace gives the same bits as the same kernels launched through spio_hip_launch with a
workspace from the allocator, on two calls in a row (the second on a smaller input, which
leaves the first call's partial sums in the rest of the shared workspace), and also matches
the fp32 CPU oracle.  The entry point is called through the C ABI (ctypes), with nothing
allocated between taking the pointers and the launches.
"""

import ctypes

import pytest
import torch

from oracle import conv2d_gw8_oracle as oracle
from spio_amd.hip import driver, get_device_attributes
from spio_amd.kernels import Conv2dGw8Params, Conv2dStats, conv2d_gw8_wgrad_kernel_factory
from spio_amd.kernels.conv2d_gw8_wgrad_kernel import Conv2dGw8WgradConfig

from helpers import gpu_args, to_gpu

pytestmark = pytest.mark.gpu

CASES = [
    # a large-filter shape whose recorded best configuration is the two-stage one, then a
    # smaller input
    (Conv2dGw8Params(n=128, c=256, h=14, w=14, padding=3, r=7, s=7),
     Conv2dGw8WgradConfig(groups=4, block_h=14, block_n=4, block_n_iters=2, two_stage=1, prefetch=2, rows=2)),
    (Conv2dGw8Params(n=6, c=40, h=20, w=19, padding=1, r=3, s=3, has_bias=True),
     Conv2dGw8WgradConfig(groups=4, block_h=7, block_n=1, block_n_iters=2, two_stage=1, prefetch=2, rows=1)),
]  # fmt: skip


def _launch_through_cabi(kernel, args, use_static):
    """The two launches of a two-stage kernel, straight through the C ABI."""
    lib = driver._load_library()
    spec = kernel.kernel_spec
    stream = torch.cuda.current_stream().cuda_stream
    workspace = None if use_static else torch.empty(spec.workspace_bytes, dtype=torch.uint8, device="cuda")
    stages = [
        (kernel.function, spec.launch_params, (workspace,) + tuple(args[1:]), 0),
        (kernel.epilogue_function, spec.epilogue_launch_params, (args[0], workspace), 1),
    ]
    for function, lp, kargs, scratch_param in stages:
        params, _keep = driver.Function.marshal(kargs)
        g, b = lp.grid, lp.block
        if use_static:
            rc = lib.spio_hip_launch_scratch(
                function.handle, g[0], g[1], g[2], b[0], b[1], b[2], lp.shared_mem_bytes,
                stream or None, params, len(kargs), scratch_param, spec.workspace_bytes)  # fmt: skip
        else:
            rc = lib.spio_hip_launch(
                function.handle, g[0], g[1], g[2], b[0], b[1], b[2], lp.shared_mem_bytes,
                stream or None, params, len(kargs))  # fmt: skip
        assert rc == 0, lib.spio_hip_last_error()
    torch.cuda.synchronize()


def test_static_workspace_matches_allocated_workspace_two_calls_in_a_row():
    attr = get_device_attributes(0)
    for params, config in CASES:
        kernel = conv2d_gw8_wgrad_kernel_factory.make_kernel(params, config, attr)
        assert kernel.kernel_spec.epilogue_suffix == "_reduce"
        assert 0 < kernel.kernel_spec.workspace_bytes <= driver.SCRATCH_BYTES
        kernel.compile()
        kernel.load(0)
        x, w, bias, dy = gpu_args(params, seed=3)
        xg, dyg = to_gpu(x), to_gpu(dy)
        outs = []
        for use_static in (False, True):
            dw = torch.zeros(params.weight_shape, device="cuda", dtype=torch.float32).contiguous(
                memory_format=torch.channels_last)  # fmt: skip
            args = [dw, xg, dyg]
            if params.has_bias:
                args.append(torch.zeros(params.c, device="cuda", dtype=torch.float32))
            torch.cuda.synchronize()
            _launch_through_cabi(kernel, args, use_static)
            outs.append(args)
        # the reduction has one owner per element and a fixed order: identical bits
        assert torch.equal(outs[0][0], outs[1][0]), f"grad_weight differs for {params.encode()}"
        _dx_e, dw_e, db_e = oracle.grads_torch(x, w, bias, dy, params.padding_h, params.padding_w)
        depth = Conv2dStats(params, output_names="grad_weight").accumulation_depths[0]
        oracle.check_close(outs[1][0], dw_e, acc_depth=depth, what=f"static-workspace wgrad {params.encode()}")
        if params.has_bias:  # grad_bias goes through fp32 atomics: equal within the tolerance
            oracle.check_close(outs[1][3], db_e, acc_depth=params.n * params.p * params.q,
                               what=f"static-workspace grad_bias {params.encode()}")  # fmt: skip
        kernel.unload()


def test_kernel_launch_with_static_workspace():
    """The same through Kernel.launch(static_workspace=True)."""
    attr = get_device_attributes(0)
    params, config = CASES[1]
    kernel = conv2d_gw8_wgrad_kernel_factory.make_kernel(params, config, attr)
    kernel.compile()
    kernel.load(0)
    x, w, bias, dy = gpu_args(params, seed=4)
    xg, dyg = to_gpu(x), to_gpu(dy)
    res = []
    for static in (False, True):
        dw = torch.zeros(params.weight_shape, device="cuda", dtype=torch.float32).contiguous(
            memory_format=torch.channels_last)  # fmt: skip
        db = torch.zeros(params.c, device="cuda", dtype=torch.float32)
        kernel.launch(dw, xg, dyg, db, static_workspace=static)
        torch.cuda.synchronize()
        res.append(dw)
    assert torch.equal(res[0], res[1])
    kernel.unload()


def test_oversized_request_is_rejected_before_any_launch():
    lib = driver._load_library()
    driver.init()
    params = (ctypes.c_void_p * 1)()
    rc = lib.spio_hip_launch_scratch(1234, 1, 1, 1, 64, 1, 1, 0, None, params, 1, 0, driver.SCRATCH_BYTES + 1)
    assert rc == 4  # SPIO_HIP_ERR_ARGUMENT
    assert b"static workspace holds" in lib.spio_hip_last_error()
    rc = lib.spio_hip_launch_scratch(1234, 1, 1, 1, 64, 1, 1, 0, None, params, 1, 3, 16)
    assert rc == 4 and b"scratch_param" in lib.spio_hip_last_error()
