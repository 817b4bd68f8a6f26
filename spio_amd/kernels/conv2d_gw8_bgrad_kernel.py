"""Fused backward kernel family of conv2d_gw8: grad_input and grad_weight in one pass.

The reference launches its data-gradient and weight-gradient kernels one after
the other (spio/functional/conv2d_gw8_function.py:119-146); both stream
grad_output.  This family reads grad_output once and produces both gradients
(and grad_bias when the params have a bias), which removes a quarter of the
backward step's HBM traffic.  The kernel computes a size-preserving convolution;
every other padding is one on a larger domain in which the input and the output
sit at fitting offsets (`bgrad_domain`).

Kernel arguments: (grad_input, grad_weight, x, grad_output, weight[, grad_bias]);
grad_weight (and grad_bias) are accumulated into, so the caller zeroes them first, unless the
configuration is two-stage (`KernelSpec.overwrites_output`): then both are stored whole.
"""

from dataclasses import dataclass, replace
from typing import Dict, List, Tuple

import torch

from ..util.math import divup
from .conv2d_gw8_kernel import _shape_defines
from .conv2d_gw8_params import Conv2dGw8Params
from .conv2d_stats import Conv2dStats
from .kernel import KernelSpec
from .kernel_factory import KernelFactory
from .launch_params import LaunchParams

SOURCE = "conv2d_gw8_bgrad_mfma.hip"

MAX_WAVES = 16
MAX_LDS_BYTES = 128 * 1024
MAX_LOADS_PER_THREAD = 4
MAX_REGISTERS = 224  # estimated fragments + accumulators + prefetch buffers, in 32-bit registers
GEOMETRIES_PER_HEIGHT = 6
MAX_UNROLLED_STEPS = 40  # SPIO_MAX_UNROLL of the kernel: longer step loops run in chunks


@dataclass(frozen=True)
class Conv2dGw8BgradConfig:
    """Tile configuration of the fused backward kernel.

    Attributes:
        groups: channel groups per workgroup (one wave each, times `split`).
        block_h: rows of grad_input (and of grad_output for the weight gradient) per
            workgroup; 0 = the whole image.  Smaller blocks give more workgroups at the price
            of re-reading the padding rows of grad_output and x at the block borders.
        block_n: images whose rows are laid side by side in one staged row.
        block_n_iters: image blocks a workgroup processes before it publishes grad_weight.
        prefetch: rows of global loads in flight ahead of the computed row (even).
        split: waves per group; they share the 32-pixel chunks (weight gradient) and the
            16-pixel tiles (data gradient) of a row.
        halo_cached: 1 = rows shared with the neighbouring row blocks are loaded with the default
            cache policy (the second reader can hit in L2), the others with the non-temporal hint.
        xcd_chunk: consecutive tiles that go to the same XCD before the next run goes to the next
            one; 0 = one contiguous range of tiles per XCD.
        two_stage: 1 = workgroups store their grad_weight (and grad_bias) sums into blocks of a
            workspace and a second kernel stores the blocks' sum into grad_weight and grad_bias,
            which then need no zero fill; 0 = workgroups add into zeroed tensors with fp32
            atomics.  Atomic additions of different workgroups to one line retire one after the
            other, and in a one-round grid all workgroups publish at the same time.
        block_q: columns per workgroup (0: the whole width; else a multiple of 32 with
            block_n = 1).  The workgroup stages block_q + S - 1 columns of x and of grad_output, so
            rows of any width fit.
    """

    groups: int = 4
    block_h: int = 0
    block_n: int = 1
    block_n_iters: int = 1
    prefetch: int = 4
    split: int = 1
    halo_cached: int = 1
    xcd_chunk: int = 4
    block_q: int = 0
    two_stage: int = 0


def bgrad_is_supported(params: Conv2dGw8Params) -> bool:
    """The fused kernel takes every shape the operator takes.

    It computes a size-preserving convolution on the domain `bgrad_domain` returns, in which the
    input and the output sit at offsets that reproduce the problem's padding.  Whether a shape
    has a legal configuration is a separate question (large filters run out of registers).
    """
    return params.r >= 1 and params.s >= 1


def bgrad_domain(params: Conv2dGw8Params) -> Tuple[int, int]:
    """Rows and columns of the images the fused kernel works on.

    The domain's own padding is r // 2 rows above (s // 2 columns left) and the rest of r - 1
    (s - 1) below (right); the input starts max(padding - r // 2, 0) rows into the domain, the
    output max(r // 2 - padding, 0), and the domain ends where the later of the two ends.
    """

    def extent(size, out_size, filt, padding):
        shift = filt // 2 - padding
        return max(max(-shift, 0) + size, max(shift, 0) + out_size)

    return (extent(params.h, params.p, params.r, params.padding_h),
            extent(params.w, params.q, params.s, params.padding_w))  # fmt: skip


def bgrad_geometry(params: Conv2dGw8Params, config: Conv2dGw8BgradConfig) -> Dict[str, int]:
    """Host mirror of the compile-time constants of conv2d_gw8_bgrad_mfma.hip."""
    r, s = params.r, params.s
    gb, nb, iters, ts, pf = config.groups, config.block_n, config.block_n_iters, config.split, config.prefetch
    dh, dw = bgrad_domain(params)
    pb, pr = r - 1 - r // 2, s - 1 - s // 2  # the domain's padding below and right
    bh = config.block_h or dh
    s2 = 2 * ((s + 1) // 2)
    nblk = s2 // 2
    bq = config.block_q or dw
    wpi = bq + s - 1
    f = nb * wpi
    kspan = (nb - 1) * wpi + bq
    kc = divup(kspan, 32)
    cpw = divup(kc, ts)
    ns = 2 * ((r + 1) // 2)
    kb = divup(s, 4)
    wt = divup(f - s + 1, 16)
    tpw = divup(wt, ts)
    fpx = 32 * kc + s2 - 1
    gsx = fpx + ((9 - fpx % 16) + 16) % 16
    fpd = max(pr + 32 * kc, 16 * wt + 4 * kb - 1)
    gsd = fpd + ((9 - fpd % 16) + 16) % 16
    nrd = 4 if (params.has_bias and r == 1) else 2 * ((r + 2) // 2)
    threads = 64 * gb * ts
    # every ring row carries a spare unit behind its last group (see the kernel)
    ring_units = 2 * (gb * gsx + 1) + nrd * (gb * gsd + 1 + ((4 - (gb * gsd + 1) % 16) + 16) % 16)
    out_row_bytes = 16 * wt * (gb * 16 + 16)
    stream_bytes = ring_units * 16 + 2 * out_row_bytes
    filter_bytes = gb * 8 * r * s * 16
    rch = r if (ts == 1 and gb * ts * r * nblk * 512 <= 96 * 1024) else 1  # RCH of the kernel
    publish_bytes = (gb * ts * rch * nblk * 128 + gb * (ts - 1) * nblk * 128 + gb * r * s * 64
                     + (gb * ts * 8 if params.has_bias else 0)) * 4  # fmt: skip
    lptx = divup(f * gb, threads)
    lptd = divup((f if config.block_q else nb * dw) * gb, threads)  # grad_output loads per row
    registers = (
        4 * ((r + 1) * nblk + 1)  # weight-gradient accumulators (+ bias)
        + 4 * tpw * (ns // 2)  # data-gradient accumulators
        + 4 * ns * kb  # filter fragments
        + 4 * (cpw * (nblk + r // 2 + 1) + tpw * kb)  # operand fragments of one step
        + 4 * pf * (lptx + lptd)  # prefetch buffers
    )
    g = dict(
        NBLK=nblk, KC=kc, CPW=cpw, WT=wt, TPW=tpw, THREADS=threads,
        LDS_BYTES=max(stream_bytes, filter_bytes, publish_bytes),
        LPTX=lptx, LPTD=lptd, REGISTERS=registers,
        STEPS=bh + pb + r - 1 + (1 if params.has_bias and r == 1 else 0),
        BH=bh, GBLKS=divup(params.groups, gb), PBLKS=divup(dh, bh), NBLKS=divup(params.n, nb * iters),
        BQ=bq, QBLKS=divup(dw, bq),
        PIXEL_EFF=(nb * bq) / (32.0 * kc),
    )  # fmt: skip
    g["NUM_BLOCKS"] = g["GBLKS"] * g["PBLKS"] * g["QBLKS"] * g["NBLKS"]
    return g


def _config_is_legal(params, config) -> bool:
    if not bgrad_is_supported(params):
        return False
    g = bgrad_geometry(params, config)
    return (
        config.groups * config.split <= MAX_WAVES
        and config.split <= min(g["KC"], g["WT"])
        and 0 <= config.block_h <= bgrad_domain(params)[0]
        and 0 <= config.block_q <= bgrad_domain(params)[1]
        and (config.block_q == 0 or (config.block_q % 32 == 0 and config.block_n == 1))
        and g["LPTD"] <= MAX_LOADS_PER_THREAD
        and config.block_n * config.block_n_iters <= max(params.n, 1)
        and g["LDS_BYTES"] <= MAX_LDS_BYTES
        and g["LPTX"] <= MAX_LOADS_PER_THREAD
        and g["REGISTERS"] <= MAX_REGISTERS
        and config.prefetch >= 2
        and config.prefetch % 2 == 0
        and config.block_n * params.c * max(params.h * params.w, params.p * params.q) * 2 < 2**31
    )


def _score(params, config, num_cus) -> float:
    """Rough relative cost used only to order (and cap) the sweep; lower is better."""
    g = bgrad_geometry(params, config)
    group_eff = params.groups / (g["GBLKS"] * config.groups)
    quant = divup(g["NUM_BLOCKS"], num_cus) * num_cus / g["NUM_BLOCKS"]
    halo = 1.0 + (2.0 / 3.0) * (params.r - 1 if g["PBLKS"] > 1 else 0) / g["BH"]
    dh, dw = bgrad_domain(params)
    stream_us = halo * 6.0 * params.n * params.c * dh * dw / 5.0e6
    publish_us = g["NUM_BLOCKS"] * config.groups * params.r * params.s * 64.0 / (128 * 2.1e3)
    split_line = 1.0 if (config.groups * 16) % 128 == 0 or config.groups == params.groups else 1.12
    return (quant * split_line / (g["PIXEL_EFF"] ** 0.3 * group_eff)) * (1.0 + publish_us / stream_us)


def _get_configs(params: Conv2dGw8Params, device_attr=None) -> List[Conv2dGw8BgradConfig]:
    """Legal configurations, most promising first; empty when the shape is not supported."""
    num_cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    G = params.groups
    # powers of two, the whole pixel, and half a pixel where the group count is not a power of two
    # (96 channels: 12 groups = 2 x 6)
    group_choices = sorted({g for g in (4, 8, 16, G, G // 2 if G % 2 == 0 and G & (G - 1) else G)
                            if 0 < g <= min(G, MAX_WAVES)}) or [min(G, MAX_WAVES)]
    # Rank the geometries of every row-block height separately and keep the best few of each:
    # whether whole images or row blocks win depends on the shape in ways the score does not
    # capture (contiguity of the channel block, halo re-reads, workgroups per compute unit).
    dh, dw = bgrad_domain(params)
    row_choices = [0] + sorted({bh for bh in (7, 14, 28) if bh < dh}, reverse=True)
    # images side by side: powers of two, and for rows shorter than a 32-pixel chunk of the weight
    # gradient's contraction the counts that fill the chunks clearly better (as in the
    # weight-gradient kernel's configuration space)
    wpi = dw + params.s - 1

    def chunk_fill(nb):
        return nb * dw / (32.0 * divup((nb - 1) * wpi + dw, 32))

    image_counts = [1, 2, 4, 8]
    if wpi < 32:
        best = max(chunk_fill(nb) for nb in image_counts)
        image_counts += [nb for nb in (3, 5, 6, 7) if chunk_fill(nb) > best + 0.05]
    # column blocks for wide rows only: narrower ones fit whole
    col_choices = [0] + [bq for bq in (64, 128) if dw >= 2 * bq and dw > 128]
    configs = []
    for bh in row_choices:
        geometries = []
        for bq in col_choices:
            for gb in group_choices:
                for nb in image_counts if bq == 0 else (1,):
                    for iters in (1, 2, 4):
                        for ts in (1, 2):
                            cfg = Conv2dGw8BgradConfig(groups=gb, block_h=bh, block_n=nb, block_n_iters=iters,
                                                       prefetch=4, split=ts, block_q=bq)  # fmt: skip
                            if _config_is_legal(params, cfg):
                                geometries.append((_score(params, cfg, num_cus), cfg))
        geometries.sort(key=lambda sc: sc[0])
        configs += [cfg for _, cfg in geometries[:GEOMETRIES_PER_HEIGHT]]
    # a shallower and a deeper pipeline for the first few: the shallow one wins where rows are short
    first = configs[:GEOMETRIES_PER_HEIGHT]
    configs += [replace(cfg, prefetch=2) for cfg in first]
    configs += [replace(cfg, prefetch=8) for cfg in first[:3] if _config_is_legal(params, replace(cfg, prefetch=8))]
    # ... and the other memory-system policies
    configs += [replace(cfg, halo_cached=hc, xcd_chunk=ch) for cfg in first[:2] for hc, ch in ((0, 4), (1, 0))]
    # ... and two-stage publishing for the leaders of every height
    configs += [replace(cfg, two_stage=1) for cfg in list(configs) if cfg.prefetch == 4 and cfg.halo_cached == 1
                and cfg.xcd_chunk == 4][:2 * GEOMETRIES_PER_HEIGHT]  # fmt: skip
    return configs


def _get_kernel_spec(params: Conv2dGw8Params, config: Conv2dGw8BgradConfig, _device_attr=None) -> KernelSpec:
    params.validate()
    assert _config_is_legal(params, config), f"illegal configuration {config} for {params}"
    g = bgrad_geometry(params, config)
    defines = _shape_defines(params)
    defines.update(SPIO_GB=config.groups, SPIO_BH=g["BH"], SPIO_NB=config.block_n,
                   SPIO_ITERS=config.block_n_iters,
                   SPIO_PF=config.prefetch, SPIO_TS=config.split,
                   SPIO_HALO_CACHED=config.halo_cached, SPIO_XCD_CHUNK=config.xcd_chunk,
                   SPIO_HAS_BIAS=int(params.has_bias))  # fmt: skip
    if config.block_q:
        defines["SPIO_BQ"] = config.block_q
    spec = KernelSpec(defines, LaunchParams(grid=g["NUM_BLOCKS"], block=g["THREADS"]), SOURCE, notes=g)
    if config.two_stage:
        # one block per workgroup: its groups' grad_weight values, then its 8 bias sums per group
        part_floats = config.groups * params.r * params.s * 64 + (config.groups * 8 if params.has_bias else 0)
        npart = g["NBLKS"] * g["PBLKS"] * g["QBLKS"]
        defines.update(SPIO_PARTIALS=1)
        spec.workspace_bytes = g["GBLKS"] * npart * part_floats * 4
        spec.workspace_arg = 1  # the workspace takes the place of grad_weight
        spec.epilogue_suffix = "_reduce"
        spec.epilogue_extra_args = (5,)  # grad_bias, or None where there is none
        spec.epilogue_launch_params = LaunchParams(grid=g["GBLKS"] * divup(part_floats // 4, 8), block=256)
        spec.overwrites_output = True
    return spec


def _make_test_args(params: Conv2dGw8Params, device):
    """Synthetic (grad_input, grad_weight, x, dy, weight[, grad_bias]) for timing."""
    cl = torch.channels_last
    x = torch.randn(params.input_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dy = torch.randn(params.output_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    w = torch.randn(params.weight_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dx = torch.empty_like(x)
    dw = torch.zeros(params.weight_shape, device=device, dtype=torch.float32).contiguous(memory_format=cl)
    if params.has_bias:
        return (dx, dw, x, dy, w, torch.zeros(params.c, device=device, dtype=torch.float32))
    return (dx, dw, x, dy, w)


conv2d_gw8_bgrad_kernel_factory = KernelFactory(
    Conv2dGw8Params,
    Conv2dGw8BgradConfig,
    Conv2dStats,
    kernel_name="spio_conv2d_gw8_bgrad",
    configs=_get_configs,
    kernel_spec=_get_kernel_spec,
    make_test_args=_make_test_args,
)
