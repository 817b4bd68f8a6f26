"""Forward / data-gradient kernel family of conv2d_gw8.

Reference: spio/kernels/conv2d_gw8_kernel.py:30-238 (`Conv2dGw8Config`,
`_get_configs`, `_get_kernel_spec`; `igrad=True` selects the data gradient,
which reuses the forward kernel with the flipped, group-transposed filter and
padding (R-1-py, S-1-px), :73-83).  The tile configuration is re-designed for
CDNA4: see csrc/conv2d_gw8_mfma.hip (row-streaming kernel) and
csrc/conv2d_gw8_image_mfma.hip (whole-image kernel for small images) for what
the fields mean on the device.
"""

from dataclasses import dataclass, replace
from math import gcd
from typing import Dict, List

import torch

from ..util.math import divup
from .conv2d_gw8_params import Conv2dGw8Params
from .conv2d_stats import Conv2dStats
from .kernel import KernelSpec
from .kernel_factory import KernelFactory
from .launch_params import LaunchParams

MFMA_SOURCE = "conv2d_gw8_mfma.hip"
IMAGE_SOURCE = "conv2d_gw8_image_mfma.hip"
DIRECT_SOURCE = "conv2d_gw8_direct.hip"

MAX_WAVES = 16
MAX_LDS_BYTES = 128 * 1024
MAX_UNROLLED_STEPS = 64  # SPIO_MAX_UNROLL of the kernel: up to here the step loop is fully unrolled
MAX_LOADS_PER_THREAD = 8
MAX_ACCUMULATORS = 16
DEVICE_LDS_BYTES = 160 * 1024
MAX_IMAGE_CONFIGS = 10  # whole-image configurations that enter the sweep
MOVER_WAVES = 4  # data-mover waves of the whole-image kernel where it has any: one per SIMD
PREFETCH_CHOICES = (2, 4, 8, 10, 12, 16)
COLUMN_BLOCK_CHOICES = (64, 128, 256)  # output columns per workgroup where rows are tiled
MAX_GEOMETRIES = 30  # tile geometries that enter the sweep; the best few also try the other cache/XCD policies


@dataclass(frozen=True)
class Conv2dGw8Config:
    """Tile configuration of the forward / data-gradient kernel.

    Attributes:
        groups: channel groups per workgroup (one wave per group and split).
        block_p: output rows per workgroup.
        block_n: images whose rows are laid side by side in one staged row.
        split: waves sharing the 16-pixel tiles of one group.
        prefetch: rows of global loads in flight ahead of the computed row.
        nontemporal: 1 = stream activations with the non-temporal hint.
        halo_cached: 1 = load rows shared with neighbouring row blocks with the default
            cache policy so the second reader can hit in L2.
        xcd_chunk: consecutive tiles that go to the same XCD (they share halo rows through its
            L2) before the next run of tiles goes to the next XCD; 0 = one contiguous range of
            tiles per XCD, 1 = tiles dealt round-robin.
        block_n_iters: whole-image kernel only: image blocks a workgroup processes one after
            the other with the same filter fragments.
        variant: "mfma" (row-streaming MFMA kernel), "image" (whole-image MFMA kernel: image
            blocks of block_n images move through LDS whole, `split` waves share a group by
            splitting its accumulators; prefetch = 2 means two LDS buffers each for input and
            output, prefetch = 1 one of each, which lets two workgroups share a CU; block_p and
            the cache/XCD policies do not apply) or "direct" (one thread per output
            pixel-group; any shape).
        movers: whole-image kernel only: extra waves that move the image blocks between global
            memory and LDS for the whole workgroup while the other waves only multiply (0: every
            wave does both).
        block_p2: row-streaming kernel only: a second tile height.  The row blocks of an image
            then alternate between block_p and block_p2 rows, the first half of the grid takes
            the block_p tiles and the second half the block_p2 tiles.  For grids of two
            workgroups per compute unit, which the device starts as two cohorts of which the
            second trails the first by the first's prefetch burst (0: one height).
        block_q: row-streaming kernel only: output columns per workgroup (0: the whole width).
            A workgroup then stages block_q + S - 1 source columns of its rows, so rows of any
            width fit (reference: block_q and block_w, spio/kernels/conv2d_gw8_kernel.py:92-108).
        prefetch_start, prefetch_rate: row-streaming kernel only: rows requested before the
            first step and per step until the requests run `prefetch` rows ahead
            (prefetch_start = 0: all `prefetch` rows at once).
    """

    groups: int = 8
    block_p: int = 16
    block_n: int = 1
    split: int = 1
    prefetch: int = 2
    variant: str = "mfma"
    nontemporal: int = 1
    halo_cached: int = 1
    xcd_chunk: int = 4
    block_n_iters: int = 1
    movers: int = 0
    block_p2: int = 0
    prefetch_start: int = 0
    prefetch_rate: int = 1
    block_q: int = 0


def direction_geometry(params: Conv2dGw8Params, igrad: bool) -> Dict[str, int]:
    """Source/destination extents and effective padding of one direction."""
    if igrad:
        return dict(SH=params.p, SW=params.q, DH=params.h, DW=params.w,
                    EPY=params.transpose_padding_h, EPX=params.transpose_padding_w)  # fmt: skip
    return dict(SH=params.h, SW=params.w, DH=params.p, DW=params.q,
                EPY=params.padding_h, EPX=params.padding_w)  # fmt: skip


def mfma_geometry(params: Conv2dGw8Params, config: Conv2dGw8Config, igrad: bool) -> Dict[str, int]:
    """Host mirror of the compile-time constants of conv2d_gw8_mfma.hip."""
    d = direction_geometry(params, igrad)
    r, s = params.r, params.s
    gb, bp, nb, ts, pf = config.groups, config.block_p, config.block_n, config.split, config.prefetch
    bp2 = config.block_p2
    bq = config.block_q or d["DW"]
    ns = 2 * ((r + 1) // 2)
    kb = (s + 3) // 4
    wpi = bq + s - 1
    f = nb * wpi
    wt = divup(f - s + 1, 16)
    fp = 16 * wt + 4 * kb - 1
    gs = fp + ((9 - fp % 16) + 16) % 16
    threads = 64 * gb * ts
    ostride = gb * 16 + 16
    lds = 2 * (gb * gs + 1) * 16 + 2 * 16 * wt * ostride  # ring rows (+ dump cell) and two output-stage rows
    if igrad:  # the data gradient stages its groups' filters in the same block first
        lds = max(lds, gb * 8 * r * s * 16)
    d.update(
        NS=ns, NACC=ns // 2, KB=kb, WPI=wpi, F=f, WT=wt, TPW=divup(wt, ts), GS=gs,
        THREADS=threads, LDS_BYTES=lds, LPT=divup(f * gb, threads),
        SPT=divup(nb * bq * gb, threads), BQ=bq, QBLKS=divup(d["DW"], bq),
        GBLKS=divup(params.groups, gb), NBLKS=divup(params.n, nb),
        # two tile heights: PBLKS (block_p, block_p2) pairs per image, one workgroup per tile
        PBLKS=divup(d["DH"], bp + bp2) if bp2 else divup(d["DH"], bp),
        STEPS=max(bp, bp2) + r - 1, UNROLL=ns // gcd(ns, pf) * pf,
    )  # fmt: skip
    d["NUM_BLOCKS"] = (2 if bp2 else 1) * d["GBLKS"] * d["PBLKS"] * d["QBLKS"] * d["NBLKS"]
    return d


def image_geometry(params: Conv2dGw8Params, config: Conv2dGw8Config, igrad: bool) -> Dict[str, int]:
    """Host mirror of the compile-time constants of conv2d_gw8_image_mfma.hip."""
    d = direction_geometry(params, igrad)
    r, s = params.r, params.s
    gb, nb, ts, iters = config.groups, config.block_n, config.split, config.block_n_iters
    ns = 2 * ((r + 1) // 2)
    nacc = ns // 2
    kb = (s + 3) // 4
    wpi = d["DW"] + s - 1
    f = nb * wpi
    wt = divup(f - s + 1, 16)
    fp = 16 * wt + 4 * kb - 1
    gs = fp + ((9 - fp % 16) + 16) % 16
    threads = 64 * (gb * ts + config.movers)
    mthreads = 64 * config.movers if config.movers else threads  # threads that move image blocks
    nbuf = 2 if config.prefetch >= 2 else 1  # prefetch = 1: single buffers (SPIO_DB = 0)
    in_units = d["SH"] * gb * gs
    out_bytes = d["DH"] * 16 * wt * (gb * 16 + 16)
    # input buffers, dump cells, output buffers (which first hold the groups' filters)
    lds = (nbuf * in_units + 32) * 16 + max(nbuf * out_bytes, gb * 8 * r * s * 16)
    lpt = divup(d["SH"] * nb * d["SW"] * gb, mthreads)
    spt = divup(d["DH"] * nb * d["DW"] * gb, mthreads)
    wlpt = divup(gb * 8 * r * s, 64 * gb * ts)  # the multiplying waves fetch the filters
    apw = max(nacc // max(ts, 1), 1)
    # registers per lane.  Multiplying: filter fragments, accumulators, two sets of source
    # fragments; moving: two blocks in flight and their LDS addresses; both: the filter share on
    # its way to LDS and the rest.  Without mover waves every wave holds both sets.
    multiplying = 4 * ns * kb + 4 * wt * apw + 8 * wt * kb
    moving = 8 * lpt + lpt + spt
    if config.movers:
        registers = max(multiplying + 4 * wlpt, moving) + 14
    else:
        registers = multiplying + 4 * max(2 * lpt, lpt + wlpt) + lpt + spt + 14
    d.update(
        NS=ns, NACC=nacc, APW=apw, KB=kb, WPI=wpi, F=f, WT=wt, GS=gs, THREADS=threads,
        MTHREADS=mthreads, LDS_BYTES=lds, LPT=lpt, SPT=spt, STEPS=d["DH"] + r - 1,
        GBLKS=divup(params.groups, gb), NBLKS=divup(params.n, nb),
        REGISTERS=registers, NBUF=nbuf,
    )  # fmt: skip
    d["WGBLKS"] = divup(d["NBLKS"], iters)
    d["NUM_BLOCKS"] = d["GBLKS"] * d["WGBLKS"]
    return d


def _image_config_is_legal(params, config, igrad) -> bool:
    g = image_geometry(params, config, igrad)
    waves = config.groups * config.split + config.movers
    # registers per lane that leave room for the workgroup's waves on a SIMD (512 in all)
    budget = {1: 232, 2: 232, 3: 160, 4: 128}.get(divup(waves, 4), 0)
    return (
        waves <= MAX_WAVES
        and config.movers >= 0
        and (config.movers == 0 or (config.prefetch >= 2 and g["MTHREADS"] % config.groups == 0))
        and g["THREADS"] % config.groups == 0
        and config.split >= 1
        and g["NACC"] % config.split == 0
        and config.block_n <= max(params.n, 1)
        and config.block_n_iters >= 1
        and g["LDS_BYTES"] <= DEVICE_LDS_BYTES
        and g["LPT"] <= MAX_LOADS_PER_THREAD
        and g["SPT"] <= MAX_LOADS_PER_THREAD
        and g["STEPS"] <= MAX_UNROLLED_STEPS
        and g["REGISTERS"] <= budget
        and config.block_n * params.c * max(params.h * params.w, params.p * params.q) * 2 < 2**31
    )


def _image_score(params, config, igrad, num_cus: int) -> float:
    """Relative cost of a whole-image configuration; lower is better.  Prices idle compute units
    (grid quantisation; LDS decides how many workgroups a CU holds), wasted MFMA columns, partial
    128-byte lines, the set-up a workgroup pays before its first block (filters through LDS,
    pipeline fill: about two blocks' worth, measured) and, weakly, split accumulators."""
    g = image_geometry(params, config, igrad)
    per_cu = max(1, min(DEVICE_LDS_BYTES // g["LDS_BYTES"], 2048 // g["THREADS"]))
    slots = num_cus * per_cu
    rounds = divup(g["NUM_BLOCKS"], slots)
    quant = rounds * slots / g["NUM_BLOCKS"]
    tile_eff = config.block_n * g["DW"] / (16.0 * g["WT"])
    group_eff = params.groups / (g["GBLKS"] * config.groups)
    split_line = 1.0 if (config.groups * 16) % 128 == 0 or config.groups == params.groups else 1.2
    setup = 1.0 + 2.0 / config.block_n_iters
    split = 1.0 + 0.05 * (config.split - 1)
    single = 1.0 if config.prefetch >= 2 else 1.03
    # mover waves pay where moving a block takes longer than multiplying it (measured: 3x3 on
    # 14x14 0.73x, 7x7 on 14x14 1.05x)
    movers = 1.0 if not config.movers else (0.9 if params.r * params.s < 25 else 1.05)
    ragged = g["WGBLKS"] * config.block_n_iters * config.block_n / params.n
    return quant * ragged * split_line * setup * split * single * movers / (tile_eff * group_eff)


def _image_configs(params: Conv2dGw8Params, igrad: bool, num_cus: int) -> List[Conv2dGw8Config]:
    """Legal whole-image configurations, most promising first (none for large images)."""
    G = params.groups
    found = []
    for gb in sorted({g for g in (4, 8, 16, G) if g <= min(G, MAX_WAVES)}):
        for nb in (1, 2, 4, 8):
            for ts in (1, 2, 4):
                for iters in (1, 2, 4, 8, 16):
                    for buffers, movers in ((2, 0), (1, 0), (2, MOVER_WAVES)):
                        cfg = Conv2dGw8Config(groups=gb, block_p=direction_geometry(params, igrad)["DH"],
                                              block_n=nb, split=ts, prefetch=buffers, variant="image",
                                              halo_cached=0, xcd_chunk=0, block_n_iters=iters,
                                              movers=movers)  # fmt: skip
                        if nb * iters > max(params.n, 1) and iters > 1:
                            continue
                        if _image_config_is_legal(params, cfg, igrad):
                            found.append((_image_score(params, cfg, igrad, num_cus), cfg))
    found.sort(key=lambda sc: sc[0])
    return [cfg for _, cfg in found[:MAX_IMAGE_CONFIGS]]


def _mfma_config_is_legal(params, config, igrad) -> bool:
    g = mfma_geometry(params, config, igrad)
    return (
        config.groups * config.split <= MAX_WAVES
        and config.split <= g["WT"]
        and config.block_n <= max(params.n, 1)
        and config.block_p <= g["DH"]
        and config.block_p2 >= 0
        and (config.block_p2 == 0 or config.block_p + config.block_p2 <= g["DH"])
        and 0 <= config.prefetch_start <= config.prefetch
        and config.prefetch_start != 1
        and config.prefetch_rate >= 1
        and 0 <= config.block_q <= g["DW"]
        and g["LDS_BYTES"] <= MAX_LDS_BYTES
        and g["LPT"] <= MAX_LOADS_PER_THREAD
        and g["TPW"] * g["NACC"] <= MAX_ACCUMULATORS
        and config.prefetch >= 2
        # the step loop is always unrolled completely (exact counts of outstanding loads/stores)
        and g["STEPS"] <= MAX_UNROLLED_STEPS
        # 32-bit buffer offsets inside a workgroup's image block
        and config.block_n * params.c * max(params.h * params.w, params.p * params.q) * 2 < 2**31
        and g["LPT"] * config.prefetch <= 24
    )


def _resident_workgroups(lds_bytes: int, threads: int) -> int:
    """Workgroups of one kernel a CU can hold (LDS and thread limits)."""
    return max(1, min(160 * 1024 // max(lds_bytes, 1), 2048 // threads, 8))


def _mfma_score(params, config, igrad, num_cus: int) -> float:
    """Rough relative cost used only to order (and cap) the sweep; lower is better.

    The kernel is HBM-bound, so the model prices extra traffic (halo rows),
    idle compute units (grid quantisation), too few bytes in flight (prefetch
    depth x resident workgroups) and, weakly, wasted MFMA columns.
    """
    g = mfma_geometry(params, config, igrad)
    halo = (config.block_p + params.r - 1) / config.block_p * (g["BQ"] + params.s - 1) / g["BQ"]
    traffic = 1.0 + 0.5 * (halo - 1.0)
    useful = config.block_n * g["BQ"]
    tile_eff = useful / (16.0 * g["WT"])
    group_eff = params.groups / (g["GBLKS"] * config.groups)
    per_cu = _resident_workgroups(g["LDS_BYTES"], g["THREADS"])
    # compute units idle in the last round of workgroups
    quant = divup(g["NUM_BLOCKS"], num_cus) * num_cus / g["NUM_BLOCKS"]
    resident = min(per_cu, max(1, g["NUM_BLOCKS"] // num_cus))
    row_bytes = g["F"] * config.groups * 16
    in_flight = resident * min(config.prefetch, g["STEPS"]) * row_bytes
    starve = 1.0 + 0.6 * max(0.0, (64 * 1024 - in_flight) / (64 * 1024))
    few_waves = 1.15 if resident * g["THREADS"] < 512 else 1.0
    # one workgroup on a CU has nothing to run while it waits at its barrier (measured at N=128,
    # C=64, 56x56: 28-row tiles, one per CU, 20.6 us; 14-row tiles, two per CU, 18.8 us)
    alone = 1.04 if resident == 1 else 1.0
    big_block = 1.08 if g["THREADS"] > 512 else 1.0
    # a workgroup that covers only part of a 128-byte line of a pixel shares it with another one
    split_line = 1.0 if (config.groups * 16) % 128 == 0 or config.groups == params.groups else 1.12
    # every row block runs block_p steps, also the last, partly empty one
    ragged = g["PBLKS"] * (config.block_p + config.block_p2) / g["DH"] * g["QBLKS"] * g["BQ"] / g["DW"]
    return traffic * quant * ragged * starve * few_waves * alone * big_block * split_line / (tile_eff ** 0.3 * group_eff)


def _two_height_configs(params, configs, igrad, num_cus) -> List[Conv2dGw8Config]:
    """Variants of the leading geometries with two tile heights, for grids that put exactly two
    workgroups on every compute unit in one round: the device starts such a grid as two cohorts
    and the second trails the first by the first's prefetch burst, so the first half of the
    grid gets taller tiles and the second half shorter ones (measured at N=128, C=64, 56x56:
    14+14 rows 18.8 us, 19+9 rows 18.3 us).  The sweep decides; they rank behind the uniform
    tiles so that a capped sweep is not spent on them."""
    out = []
    seen = set()
    for cfg in configs:
        shape = (cfg.groups, cfg.block_p, cfg.block_n, cfg.split)
        if len(seen) == 2 or shape in seen:
            continue
        g = mfma_geometry(params, cfg, igrad)
        if cfg.variant != "mfma" or cfg.block_p2 or g["NUM_BLOCKS"] != 2 * num_cus:
            continue
        if g["PBLKS"] % 2 or g["DH"] % (2 * cfg.block_p) or cfg.block_p < 4:
            continue
        seen.add(shape)
        for frac in (0.29, 0.36, 0.43):
            delta = max(1, round(cfg.block_p * frac))
            for pf in sorted({cfg.prefetch, 10, 12}):
                cand = replace(cfg, block_p=cfg.block_p + delta, block_p2=cfg.block_p - delta, prefetch=pf)
                if cand not in out and _mfma_config_is_legal(params, cand, igrad):
                    out.append(cand)
    return out


def _get_configs(params: Conv2dGw8Params, device_attr=None, igrad: bool = False) -> List[Conv2dGw8Config]:
    """Legal configurations, most promising first; the direct kernel is always last."""
    d = direction_geometry(params, igrad)
    num_cus = getattr(device_attr, "multiprocessor_count", 256) or 256
    G = params.groups
    group_choices = sorted({g for g in (4, 8, 16, G) if g <= min(G, MAX_WAVES)}) or [min(G, MAX_WAVES)]
    row_choices = sorted({bp for bp in (2, 4, 7, 8, 14, 16, 28, 32, 56, d["DH"]) if bp <= d["DH"]})
    # column blocks for wide rows only: narrower ones fit whole and pay no column halo
    col_choices = [0] + [bq for bq in COLUMN_BLOCK_CHOICES if d["DW"] >= 2 * bq and d["DW"] > 128]
    found = []
    for bq in col_choices:
        for gb in group_choices:
            for nb in (1, 2, 4, 8) if bq == 0 else (1,):
                for ts in (1, 2, 4):
                    for bp in row_choices:
                        steps = bp + params.r - 1
                        for pf in PREFETCH_CHOICES:
                            if pf > 2 and pf > steps:
                                continue
                            cfg = Conv2dGw8Config(groups=gb, block_p=bp, block_n=nb, split=ts, prefetch=pf, block_q=bq)
                            if _mfma_config_is_legal(params, cfg, igrad):
                                found.append((_mfma_score(params, cfg, igrad, num_cus), cfg))
    found.sort(key=lambda sc: sc[0])
    configs = [cfg for _, cfg in found[:MAX_GEOMETRIES]]
    # the memory-system policies, which the score cannot rank: halo rows with or without the
    # non-temporal hint, and how tiles are dealt to the XCDs
    leading = []  # the first four tile geometries, whatever their prefetch depth
    for cfg in configs:
        shape = (cfg.groups, cfg.block_p, cfg.block_n, cfg.split)
        if shape not in leading:
            if len(leading) == 4:
                break
            leading.append(shape)
    for cfg in list(configs):
        if (cfg.groups, cfg.block_p, cfg.block_n, cfg.split) in leading:
            for hc, ch in ((0, 4), (1, 0), (0, 0)):
                configs.append(replace(cfg, halo_cached=hc, xcd_chunk=ch))
    configs += _two_height_configs(params, configs, igrad, num_cus)
    # small images: the whole-image kernel; its two best candidates go first, so that the capped
    # sweep an operator runs on an unrecorded shape sees both kernels
    image = _image_configs(params, igrad, num_cus)
    if image and image_geometry(params, image[0], igrad)["NUM_BLOCKS"] >= num_cus:
        configs = image[:2] + configs + image[2:]
    else:  # too few image blocks to fill the device with workgroups that each pay the set-up
        configs = configs[:2] + image[:2] + configs[2:] + image[2:]
    configs.append(Conv2dGw8Config(groups=1, block_p=1, block_n=1, split=1, variant="direct"))
    return configs


def _shape_defines(params: Conv2dGw8Params) -> Dict[str, object]:
    return {
        "SPIO_N": params.n, "SPIO_C": params.c, "SPIO_H": params.h, "SPIO_W": params.w,
        "SPIO_R": params.r, "SPIO_S": params.s,
        "SPIO_PY": params.padding_h, "SPIO_PX": params.padding_w,
    }  # fmt: skip


def _get_kernel_spec(params: Conv2dGw8Params, config: Conv2dGw8Config, _device_attr=None,
                     igrad: bool = False) -> KernelSpec:  # fmt: skip
    """Macros and launch geometry for one (params, config, direction)."""
    params.validate()
    defines = _shape_defines(params)
    defines["SPIO_IGRAD"] = int(igrad)
    defines["SPIO_HAS_BIAS"] = int(params.has_bias and not igrad)
    if config.variant == "direct":
        d = direction_geometry(params, igrad)
        threads = 256
        defines["SPIO_BLOCK_THREADS"] = threads
        total = params.n * d["DH"] * d["DW"] * params.groups
        return KernelSpec(defines, LaunchParams(grid=divup(total, threads), block=threads), DIRECT_SOURCE)
    if config.variant == "image":
        assert _image_config_is_legal(params, config, igrad), f"illegal configuration {config} for {params}"
        g = image_geometry(params, config, igrad)
        defines.update(
            SPIO_GB=config.groups, SPIO_NB=config.block_n, SPIO_TS=config.split,
            SPIO_ITERS=config.block_n_iters, SPIO_NT=config.nontemporal,
            SPIO_DB=int(config.prefetch >= 2), SPIO_MV=config.movers,
        )  # fmt: skip
        return KernelSpec(
            defines, LaunchParams(grid=g["NUM_BLOCKS"], block=g["THREADS"]), IMAGE_SOURCE, notes=g
        )
    if config.variant != "mfma":
        raise ValueError(f"unknown kernel variant {config.variant!r}")
    assert _mfma_config_is_legal(params, config, igrad), f"illegal configuration {config} for {params}"
    g = mfma_geometry(params, config, igrad)
    defines.update(
        SPIO_GB=config.groups, SPIO_BP=config.block_p, SPIO_NB=config.block_n,
        SPIO_TS=config.split, SPIO_PF=config.prefetch,
        SPIO_NT=config.nontemporal, SPIO_HALO_CACHED=config.halo_cached,
        SPIO_XCD_CHUNK=config.xcd_chunk,
    )  # fmt: skip
    if config.block_p2:
        defines["SPIO_BP2"] = config.block_p2
    if config.prefetch_start:
        defines["SPIO_PF0"] = config.prefetch_start
    if config.prefetch_rate != 1:
        defines["SPIO_PF_RATE"] = config.prefetch_rate
    if config.block_q:
        defines["SPIO_BQ"] = config.block_q
    return KernelSpec(
        defines, LaunchParams(grid=g["NUM_BLOCKS"], block=g["THREADS"]), MFMA_SOURCE, notes=g
    )


def _get_kernel_name(igrad: bool = False) -> str:
    return "spio_conv2d_gw8_dgrad" if igrad else "spio_conv2d_gw8_fprop"


def _make_test_args(params: Conv2dGw8Params, device, igrad: bool = False):
    """Synthetic (dst, src, weight, bias) for timing."""
    cl = torch.channels_last
    x = torch.randn(params.input_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    y = torch.randn(params.output_shape, device=device, dtype=torch.float16).contiguous(memory_format=cl)
    w = (torch.randn(params.weight_shape, device=device, dtype=torch.float16) * 0.1).contiguous(memory_format=cl)
    if igrad:
        return (x, y, w, None)
    bias = torch.randn(params.bias_shape, device=device, dtype=torch.float32) if params.has_bias else None
    return (y, x, w, bias)


conv2d_gw8_kernel_factory = KernelFactory(
    Conv2dGw8Params,
    Conv2dGw8Config,
    Conv2dStats,
    kernel_name=_get_kernel_name,
    configs=_get_configs,
    kernel_spec=_get_kernel_spec,
    make_test_args=_make_test_args,
)
