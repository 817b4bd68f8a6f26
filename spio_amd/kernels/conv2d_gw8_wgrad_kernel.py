"""Weight-gradient kernel family of conv2d_gw8.

Kernel arguments: (grad_weight, x, grad_output) and, when the params have a
bias, a fourth `grad_bias` ([K] fp32, pre-zeroed like grad_weight, or None):
the kernels then also sum grad_output per channel in the same pass, which the
reference leaves to a separate reduction (spio/functional/conv2d_gw8_function.py:134-136).

Reference: spio/kernels/conv2d_gw8_wgrad_kernel.py:27-285.  The kernel adds
its partial sums into a pre-zeroed fp32 tensor laid out [K][R][S][8]
(spio/functional/conv2d_gw8_function.py:124-130).
"""

from dataclasses import dataclass, replace
from typing import Dict, List

import torch

from ..util.math import divup
from .conv2d_gw8_kernel import _shape_defines
from .conv2d_gw8_params import Conv2dGw8Params
from .conv2d_stats import Conv2dStats
from .kernel import KernelSpec
from .kernel_factory import KernelFactory
from .launch_params import LaunchParams

DIRECT_SOURCE = "conv2d_gw8_direct.hip"
MFMA_SOURCE = "conv2d_gw8_wgrad_mfma.hip"

MAX_WAVES = 16
MAX_LDS_BYTES = 128 * 1024
MAX_LOADS_PER_THREAD = 8
MAX_ACCUMULATORS = 32
MAX_GEOMETRIES = 16
PIPELINE_CHOICES = ((2, 1, 0), (4, 1, 0), (2, 2, 0), (2, 1, 1), (4, 1, 1))  # (prefetch, rows, pipe)


@dataclass(frozen=True)
class Conv2dGw8WgradConfig:
    """Tile configuration of the weight-gradient kernel.

    Attributes:
        groups: channel groups (waves) per workgroup.
        block_h: rows of grad_output per workgroup.
        block_n: images whose rows are laid side by side in one staged row.
        block_n_iters: image blocks a workgroup accumulates before its atomics.
        chunks: (direct variant only) pixel chunks per group.
        prefetch: steps of global loads in flight ahead of the computed step (even).
        rows: rows of x (and of grad_output) a workgroup multiplies between two barriers,
            1 or 2; two rows share their grad_output fragments and halve the barriers at the
            price of a deeper LDS ring.
        split: waves sharing the 32-pixel chunks of one group; their sums are added in LDS
            before publishing, so bigger workgroups do not publish more.
        two_stage: 1 = workgroups store partial sums to a workspace and a second kernel
            stores their sum into grad_weight (no zero fill needed, deterministic); 0 =
            workgroups add into a zeroed grad_weight with fp32 atomics.
        variant: "mfma" (row-streaming MFMA kernel) or "direct" (any shape).
        block_q: grad_output columns per workgroup (0: the whole width); the workgroup stages
            block_q + S - 1 columns of x opposite them, so rows of any width fit.
        pipe: 1 = the MFMAs of a step are issued one step later, from a second set of fragment
            registers, with the next step's LDS reads, row loads and ring writes dealt out
            between them; 0 = every step reads its fragments, then multiplies.
    """

    groups: int = 8
    block_h: int = 14
    block_n: int = 1
    block_n_iters: int = 1
    chunks: int = 0
    variant: str = "mfma"
    prefetch: int = 2
    two_stage: int = 0
    split: int = 1
    rows: int = 1
    block_q: int = 0
    pipe: int = 0


def image_placement(params: Conv2dGw8Params, nb: int, block_q: int = 0) -> Dict[str, int]:
    """Where the images of a staged row sit (mirror of the kernel's constants).

    Images follow one another GAP = max(px, S-1-px) zero cells apart (the right halo of one is
    the left halo of the next).  The contraction runs over 32-pixel chunks of the grad_output
    row; where a chunk holds whole images and that takes fewer chunks than the images laid end
    to end, every chunk gets its own images (PACKED).
    """
    s, px = params.s, params.padding_w
    s2 = 2 * ((s + 1) // 2)
    bq = block_q or params.q
    gap = max(px, s - 1 - px)
    ip = bq + s - 1 if block_q else bq + gap
    ipc_max = (32 + ip - bq) // ip
    kc_flat = divup((nb - 1) * ip + bq, 32)
    kc_packed = divup(nb, ipc_max) if ipc_max > 0 else kc_flat
    packed = kc_packed < kc_flat
    kc = kc_packed if packed else kc_flat
    xcp = 16 * divup(32 + s2 - 1, 16) if packed else 32
    return dict(IP=ip, IPC=ipc_max if packed else nb, KC=kc, PACKED=int(packed), XCP=xcp,
                FPX=kc * xcp if packed else 32 * kc + s2 - 1)  # fmt: skip


def wgrad_geometry(params: Conv2dGw8Params, config: Conv2dGw8WgradConfig) -> Dict[str, int]:
    """Host mirror of the compile-time constants of conv2d_gw8_wgrad_mfma.hip."""
    r, s = params.r, params.s
    gb, bh, nb, iters, ts = config.groups, config.block_h, config.block_n, config.block_n_iters, config.split
    s2 = 2 * ((s + 1) // 2)
    bq = config.block_q or params.q
    wpi = bq + s - 1
    f = nb * wpi
    place = image_placement(params, nb, config.block_q)
    kc, fpx = place["KC"], place["FPX"]
    gsx = fpx + ((9 - fpx % 16) + 16) % 16
    fpd = 32 * kc
    gsd = fpd + ((9 - fpd % 16) + 16) % 16
    rb = config.rows
    nrx = 2 * rb
    nrd = (4 if (params.has_bias and r == 1) else 2 * ((r + 2) // 2)) + (2 if rb == 2 else 0)
    threads = 64 * gb * ts
    lds_rings = (nrx * gb * gsx + nrd * (gb * gsd + ((4 - (gb * gsd) % 16) + 16) % 16)) * 16
    # the same LDS block holds the reduction scratch at the end: per-wave row-slot halves, the
    # sums of the other waves of a split group, and (atomic publishing) every group's R*S*64 sums
    rch = r if (ts == 1 and gb * ts * r * (s2 // 2) * 512 <= 96 * 1024) else 1  # RCH of the kernel
    lds_scratch = (gb * ts * rch * (s2 // 2) * 128 + gb * (ts - 1) * (s2 // 2) * 128
                   + (0 if config.two_stage else gb * r * s * 64)
                   + (gb * ts * 8 if params.has_bias else 0)) * 4  # fmt: skip
    g = dict(
        NBLK=s2 // 2, ND=r + 1, WPI=wpi, F=f, KC=kc, GSX=gsx, GSD=gsd, NRD=nrd, THREADS=threads,
        LDS_BYTES=max(lds_rings, lds_scratch), RING_BYTES=lds_rings, SCRATCH_BYTES=lds_scratch,
        LPTX=divup(f * gb, threads), LPTD=divup(nb * bq * gb, threads),
        BQ=bq, QBLKS=divup(params.q, bq),
        GBLKS=divup(params.groups, gb), PBLKS=divup(params.p, bh),
        NBLKS=divup(params.n, nb * iters),
        STEPS=divup(bh + (2 if params.has_bias and r == 1 else r) - 1, rb),
        PIXEL_EFF=(nb * bq) / (32.0 * kc), IPC=place["IPC"], PACKED=place["PACKED"],
    )  # fmt: skip
    g["NUM_BLOCKS"] = g["GBLKS"] * g["PBLKS"] * g["QBLKS"] * g["NBLKS"]
    return g


def _mfma_config_is_legal(params, config) -> bool:
    g = wgrad_geometry(params, config)
    return (
        config.groups * config.split <= MAX_WAVES
        and config.split <= g["KC"]
        and config.block_h <= params.p
        and config.block_n * config.block_n_iters <= max(params.n, 1)
        and g["LDS_BYTES"] <= MAX_LDS_BYTES
        and g["LPTX"] <= MAX_LOADS_PER_THREAD
        and g["ND"] * g["NBLK"] <= MAX_ACCUMULATORS
        and config.prefetch >= 2
        and config.prefetch % 2 == 0
        and config.rows in (1, 2)
        and config.pipe in (0, 1)
        and 0 <= config.block_q <= params.q
        and (g["LPTX"] + g["LPTD"]) * config.prefetch * config.rows <= 32
        # the kernel indexes both tensors in 16-byte units with 32-bit integers
        and params.n * params.groups * max(params.h * params.w, params.p * params.q) < 2**31
    )


def _mfma_score(params, config, num_cus) -> float:
    """Rough relative cost used only to order (and cap) the sweep; lower is better."""
    g = wgrad_geometry(params, config)
    halo = (config.block_h + params.r - 1) / config.block_h
    traffic = 1.0 + 0.5 * (halo - 1.0) + 0.25 * (params.s - 1) / g["BQ"]
    group_eff = params.groups / (g["GBLKS"] * config.groups)
    # compute units idle in the last round of workgroups
    quant = divup(g["NUM_BLOCKS"], num_cus) * num_cus / g["NUM_BLOCKS"]
    # Publishing costs R*S*64 values per (workgroup, group): atomics retire at roughly 128 per
    # clock device-wide; partial stores plus the reduction kernel cost bandwidth and a launch.
    stream_bytes = 4.0 * params.n * params.c * params.h * params.w
    stream_us = stream_bytes / 5.0e6
    values = g["NUM_BLOCKS"] * config.groups * params.r * params.s * 64.0
    if config.two_stage:
        publish_us = 4.5 + 2.0 * 4.0 * values / 5.0e6
    else:
        publish_us = values / (128 * 2.1e3)
    split_line = 1.0 if (config.groups * 16) % 128 == 0 or config.groups == params.groups else 1.12
    return (traffic * quant * split_line / (g["PIXEL_EFF"] ** 0.3 * group_eff)) * (
        1.0 + publish_us / stream_us
    )


def _get_configs(params: Conv2dGw8Params, device_attr=None) -> List[Conv2dGw8WgradConfig]:
    """Legal configurations, most promising first; a direct-kernel configuration closes the list."""
    num_cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    G = params.groups
    # powers of two, the whole pixel, and half a pixel where the group count is not a power of two
    # (96 channels: 12 groups = 2 x 6)
    group_choices = sorted({g for g in (4, 8, 16, G, G // 2 if G % 2 == 0 and G & (G - 1) else G)
                            if 0 < g <= min(G, MAX_WAVES)}) or [min(G, MAX_WAVES)]
    row_choices = sorted({bh for bh in (4, 7, 8, 14, 16, 28, 32, 56, params.p) if bh <= params.p})
    # Images side by side.  The contraction runs over 32-pixel chunks of the flattened row, so
    # where a padded image row is shorter than a chunk the count decides how full the chunks
    # are: besides the powers of two, the counts that fill them clearly better (7x7 images with
    # one halo column each side: 8 images fill 56 of 96 pixels, 7 images 49 of 64).
    def chunk_fill(nb):
        return nb * params.q / (32.0 * image_placement(params, nb)["KC"])

    image_counts = [1, 2, 4, 8]
    if params.q + params.s - 1 < 32:
        best = max(chunk_fill(nb) for nb in image_counts)
        image_counts += [nb for nb in (3, 5, 6, 7) if chunk_fill(nb) > best + 0.05]
    # Rank the tile geometries first and keep the best few; each of them is then tried with the
    # pipeline variants (prefetch distance, rows per step), which the score cannot tell apart.
    # column blocks for wide rows only: narrower ones fit whole
    col_choices = [0] + [bq for bq in (64, 128, 256) if params.q >= 2 * bq and params.q > 128]
    geometries = []
    for bq in col_choices:
        for gb in group_choices:
            for nb in image_counts if bq == 0 else (1,):
                for iters in (1, 2, 4, 8):
                    for bh in row_choices:
                        for two_stage in (0, 1):
                            for ts in (1, 2):
                                cfg = Conv2dGw8WgradConfig(groups=gb, block_h=bh, block_n=nb, block_n_iters=iters,
                                                           prefetch=2, two_stage=two_stage, split=ts, block_q=bq)  # fmt: skip
                                if _mfma_config_is_legal(params, cfg):
                                    geometries.append((_mfma_score(params, cfg, num_cus), cfg))
    geometries.sort(key=lambda sc: sc[0])
    configs = []
    for _, base in geometries[:MAX_GEOMETRIES]:
        for pf, rows, pipe in PIPELINE_CHOICES:
            if pf > 2 and pf * rows > base.block_h + params.r - 1:
                continue
            cfg = replace(base, prefetch=pf, rows=rows, pipe=pipe)
            if _mfma_config_is_legal(params, cfg):
                configs.append(cfg)
    total_pix = params.n * params.p * params.q
    chunks = max(1, min(divup(8 * num_cus, params.groups), divup(total_pix, 64)))
    configs.append(Conv2dGw8WgradConfig(groups=1, block_h=1, block_n=1, block_n_iters=1,
                                        chunks=chunks, variant="direct"))  # fmt: skip
    return configs


def _get_kernel_spec(params: Conv2dGw8Params, config: Conv2dGw8WgradConfig, _device_attr=None) -> KernelSpec:
    params.validate()
    defines = _shape_defines(params)
    # with a bias the kernels take a fourth pointer and also accumulate grad_bias
    defines["SPIO_HAS_BIAS"] = int(params.has_bias)
    if config.variant == "direct":
        threads = 256
        defines.update(SPIO_WGRAD=1, SPIO_BLOCK_THREADS=threads, SPIO_WGRAD_CHUNKS=config.chunks)
        return KernelSpec(
            defines, LaunchParams(grid=params.groups * config.chunks, block=threads), DIRECT_SOURCE
        )
    if config.variant != "mfma":
        raise ValueError(f"unknown kernel variant {config.variant!r}")
    assert _mfma_config_is_legal(params, config), f"illegal configuration {config} for {params}"
    g = wgrad_geometry(params, config)
    defines.update(SPIO_GB=config.groups, SPIO_BH=config.block_h, SPIO_NB=config.block_n,
                   SPIO_ITERS=config.block_n_iters, SPIO_PF=config.prefetch,
                   SPIO_TS=config.split, SPIO_RB=config.rows)  # fmt: skip
    if config.pipe:
        defines["SPIO_PIPE"] = 1
    if config.block_q:
        defines["SPIO_BQ"] = config.block_q
    spec = KernelSpec(defines, LaunchParams(grid=g["NUM_BLOCKS"], block=g["THREADS"]), MFMA_SOURCE, notes=g)
    if config.two_stage:
        num_partials = g["NBLKS"] * g["PBLKS"] * g["QBLKS"]
        # float4 columns of the partial blocks of one (image block, row block): per wave
        # [r][tap pair][4][32 lanes] floats
        cols = g["GBLKS"] * config.groups * params.r * g["NBLK"] * 32
        defines.update(SPIO_PARTIALS=1)
        spec.workspace_bytes = num_partials * cols * 16
        spec.epilogue_suffix = "_reduce"
        spec.overwrites_output = True  # the second stage stores grad_weight whole
        # one workgroup per 32 float4 columns (cols is a multiple of 32 per channel block)
        spec.epilogue_launch_params = LaunchParams(grid=cols // 32, block=256)
    return spec


def _make_test_args(params: Conv2dGw8Params, device):
    """Synthetic (grad_weight, x, dy[, grad_bias]) for timing."""
    cl = torch.channels_last
    x = torch.randn(params.input_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dy = torch.randn(params.output_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    dw = torch.zeros(params.weight_shape, device=device, dtype=torch.float32).contiguous(memory_format=cl)
    if params.has_bias:
        return (dw, x, dy, torch.zeros(params.c, device=device, dtype=torch.float32))
    return (dw, x, dy)


conv2d_gw8_wgrad_kernel_factory = KernelFactory(
    Conv2dGw8Params,
    Conv2dGw8WgradConfig,
    Conv2dStats,
    kernel_name="spio_conv2d_gw8_wgrad",
    configs=_get_configs,
    kernel_spec=_get_kernel_spec,
    make_test_args=_make_test_args,
)
