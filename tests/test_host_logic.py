"""Host-side kernel infrastructure without a GPU: configuration spaces, launch
geometry, JIT specialisation of every kernel family, caches and the tuner's
record store.  CPU only."""

import json
import os

import pytest

from helpers import reference_test_params
from spio_amd.hip import DeviceAttributes
from spio_amd.kernels import (
    Conv2dGw8Config,
    Conv2dGw8Params,
    KernelCache,
    KernelFactory,
    KernelKey,
    KernelParamsLogger,
    LaunchParams,
    conv2d_gw8_bgrad_kernel_factory,
    conv2d_gw8_kernel_factory,
    conv2d_gw8_wgrad_kernel_factory,
    kernel_params_logging_is_enabled,
)
from spio_amd.kernels.conv2d_gw8_kernel import MAX_LDS_BYTES, image_geometry, mfma_geometry
from spio_amd.kernels.tuner import Tuner, device_key

ATTR = DeviceAttributes()


def test_launch_params_normalisation():
    lp = LaunchParams(grid=7, block=(64, 2))
    assert lp.grid == (7, 1, 1) and lp.block == (64, 2, 1)
    with pytest.raises(AssertionError):
        LaunchParams(grid=0, block=64)
    with pytest.raises(ValueError):
        LaunchParams(grid=(1, 1, 1, 1), block=64)


@pytest.mark.parametrize("igrad", [False, True])
def test_every_shape_has_legal_configs(igrad):
    """Every shape of the reference's test list gets configurations whose derived
    geometry respects the device limits, and the direct kernel closes the list."""
    for params in reference_test_params(False):
        configs = conv2d_gw8_kernel_factory.configs(params, ATTR, igrad=igrad)
        assert configs and configs[-1].variant == "direct"
        assert len(set(configs)) == len(configs)
        for cfg in configs[:-1]:
            if cfg.variant == "image":  # the whole-image kernel has its own geometry
                g = image_geometry(params, cfg, igrad)
                assert g["THREADS"] <= 1024 and g["LDS_BYTES"] <= 160 * 1024 and g["NACC"] % cfg.split == 0
                spec = conv2d_gw8_kernel_factory.get_kernel_spec(params, cfg, ATTR, igrad=igrad)
                assert spec.launch_params.grid[0] == g["NUM_BLOCKS"] == g["GBLKS"] * g["WGBLKS"]
                assert spec.launch_params.block[0] == g["THREADS"]
                assert g["WGBLKS"] * cfg.block_n_iters * cfg.block_n >= params.n
                # data-mover waves come on top of the multiplying waves, need the second pair of
                # buffers, and a moving thread stays with one group
                assert g["THREADS"] == 64 * (cfg.groups * cfg.split + cfg.movers)
                assert g["MTHREADS"] == (64 * cfg.movers if cfg.movers else g["THREADS"])
                assert g["MTHREADS"] % cfg.groups == 0
                assert spec.defines["SPIO_MV"] == cfg.movers
                if cfg.movers:
                    assert cfg.prefetch >= 2 and spec.defines["SPIO_DB"] == 1
                continue
            g = mfma_geometry(params, cfg, igrad)
            assert g["THREADS"] <= 1024 and g["LDS_BYTES"] <= MAX_LDS_BYTES
            assert g["NUM_BLOCKS"] >= 1 and g["WT"] * 16 >= g["F"] - params.s + 1
            assert g["GS"] % 16 == 9 and g["GS"] >= 16 * g["WT"] + 4 * g["KB"] - 1
            spec = conv2d_gw8_kernel_factory.get_kernel_spec(params, cfg, ATTR, igrad=igrad)
            assert spec.launch_params.grid[0] == g["NUM_BLOCKS"]
            assert spec.launch_params.block[0] == g["THREADS"]


def test_model_shapes_and_wide_rows_get_mfma_kernels(capsys):
    """No performance cliff onto the any-shape kernel: every model-derived shape (at its full
    batch) and rows of any width (column blocks: 224, 384, 512, 1024 and 4000 pixels) have an
    MFMA configuration in every family, the fused backward kernel included for 3x3 and 5x5
    filters; a request that has only the any-shape kernel says so on first use."""
    from helpers import GOLDEN

    with open(os.path.join(GOLDEN, "conv2d_gw8_model_shapes.json"), encoding="utf-8") as f:
        rows = json.load(f)
    shapes = [Conv2dGw8Params(n=d["n"], c=d["c"], h=d["h"], w=d["w"], padding=(d["py"], d["px"]),
                              r=d["r"], s=d["s"], has_bias=d["has_bias"]) for d in rows]  # fmt: skip
    shapes += [Conv2dGw8Params(n=8, c=c, h=64, w=w) for c in (64, 256) for w in (64, 96, 128)]
    shapes += [Conv2dGw8Params(n=8, c=256, h=64, w=64, r=7, s=7, padding=3)]
    wide = [Conv2dGw8Params(n=2, c=c, h=20, w=w, r=r, s=r, padding=r // 2, has_bias=b)
            for w in (224, 384, 512, 1024, 4000) for c, r, b in ((64, 3, False), (32, 5, True), (256, 3, True))]  # fmt: skip
    wide += [Conv2dGw8Params(n=2, c=64, h=20, w=w, r=7, s=7, padding=3) for w in (224, 512, 1024)]
    for params in shapes + wide:
        for factory, kw in ((conv2d_gw8_kernel_factory, {}), (conv2d_gw8_kernel_factory, {"igrad": True}),
                            (conv2d_gw8_wgrad_kernel_factory, {})):  # fmt: skip
            configs = factory.configs(params, ATTR, **kw)
            assert any(c.variant == "mfma" for c in configs), f"{factory.get_full_kernel_name(params, **kw)}: direct only"
    for params in wide:
        if params.r <= 5:
            configs = list(conv2d_gw8_bgrad_kernel_factory.configs(params, ATTR))
            assert configs and all(c.block_q % 32 == 0 for c in configs), f"fused backward: none for {params.encode()}"
            if params.w >= 512:
                assert all(c.block_q > 0 for c in configs)

    # the cliff is announced where a request has nothing but the any-shape kernel
    huge = Conv2dGw8Params(n=1, c=64, h=8, w=4000)
    direct_only = KernelFactory(Conv2dGw8Params, Conv2dGw8Config, None, kernel_name="spio_conv2d_gw8_fprop",
                                configs=lambda p, a: [Conv2dGw8Config(variant="direct")],
                                kernel_spec=None)  # fmt: skip

    class Stop(Exception):
        pass

    def no_compile(*a, **k):
        raise Stop

    import spio_amd.kernels.kernel_cache as kernel_cache

    saved = kernel_cache.compile_and_load_kernel
    kernel_cache.compile_and_load_kernel = no_compile
    try:
        with pytest.raises(Stop):
            Tuner().best_kernel(direct_only, huge, 0, ATTR)
    finally:
        kernel_cache.compile_and_load_kernel = saved
    assert "no MFMA configuration fits" in capsys.readouterr().err


def test_kernel_names_follow_the_reference_convention():
    p = Conv2dGw8Params(n=4, c=64, h=16, w=32, has_bias=True)
    f = conv2d_gw8_kernel_factory
    assert f.get_full_kernel_name(p) == "spio_conv2d_gw8_fprop__4n_64c_16h_32w_1py_1px_3r_3s_b"
    assert f.get_full_kernel_name(p, igrad=True).startswith("spio_conv2d_gw8_dgrad__")
    assert conv2d_gw8_wgrad_kernel_factory.get_full_kernel_name(p).startswith("spio_conv2d_gw8_wgrad__")
    assert f.get_kernel_cache() is f.get_kernel_cache()
    assert f.get_kernel_cache() is not f.get_kernel_cache(igrad=True)


@pytest.mark.parametrize(
    "params",
    [
        Conv2dGw8Params(n=4, c=64, h=16, w=32, has_bias=True),
        Conv2dGw8Params(n=3, c=24, h=20, w=19, padding=(2, 0), r=4, s=1),
        Conv2dGw8Params(n=2, c=32, h=14, w=14, padding=3, r=7, s=7),
        Conv2dGw8Params(n=3, c=24, h=20, w=19, padding=(0, 2)),
    ],
    ids=lambda p: p.encode(),
)
def test_jit_specialisation_of_every_family(params):
    """hipRTC compiles first/last configuration of each family for gfx950 (no GPU needed)."""
    for factory, kw in ((conv2d_gw8_kernel_factory, {}), (conv2d_gw8_kernel_factory, {"igrad": True}),
                        (conv2d_gw8_wgrad_kernel_factory, {}), (conv2d_gw8_bgrad_kernel_factory, {})):  # fmt: skip
        configs = list(factory.configs(params, ATTR, **kw))
        if not configs:  # the fused backward kernel has no configuration for 7x7 (registers)
            assert factory is conv2d_gw8_bgrad_kernel_factory
            continue
        for cfg in {configs[0], configs[-1]}:
            kernel = factory.make_kernel(params, cfg, ATTR, **kw)
            kernel.compile()
            assert kernel.code[:4] == b"\x7fELF"
            assert kernel.kernel_name.encode() in kernel.code
            with pytest.raises(ValueError):
                kernel.launch()  # not loaded


def test_packaged_tuning_records_name_configurations_that_still_exist():
    """A packaged record whose configuration is no longer a candidate would be ignored and
    trigger a sweep on first use; keep the records in step with the configuration spaces."""
    import dataclasses
    import os

    import spio_amd.kernels as kernels_pkg

    from spio_amd.kernels import LayerNorm2dParams, layernorm_2d_bwd_kernel_factory, layernorm_2d_kernel_factory

    families = {
        "spio_conv2d_gw8_fprop": (conv2d_gw8_kernel_factory, {}),
        "spio_conv2d_gw8_dgrad": (conv2d_gw8_kernel_factory, {"igrad": True}),
        "spio_conv2d_gw8_wgrad": (conv2d_gw8_wgrad_kernel_factory, {}),
        "spio_conv2d_gw8_bgrad": (conv2d_gw8_bgrad_kernel_factory, {}),
        "spio_layernorm_2d": (layernorm_2d_kernel_factory, {}),
        "spio_layernorm_2d_bwd": (layernorm_2d_bwd_kernel_factory, {}),
    }
    tuned = os.path.join(os.path.dirname(kernels_pkg.__file__), "tuned")
    checked = 0
    for fname in os.listdir(tuned):
        arch, cus = fname[: -len(".json")].rsplit("_", 1)
        attr = dataclasses.replace(DeviceAttributes(), arch=arch, multiprocessor_count=int(cus[:-2]))
        with open(os.path.join(tuned, fname), encoding="utf-8") as f:
            records = json.load(f)
        for key, record in records.items():
            name, encoded = key.split("__")
            factory, kw = families[name]
            params = (LayerNorm2dParams if name.startswith("spio_layernorm_2d") else Conv2dGw8Params).decode(encoded)
            config = factory.config_cls(**record["config"])
            assert config in list(factory.configs(params, attr, **kw)), f"stale record {key}: {config}"
            assert record["us"] > 0
            checked += 1
    assert checked > 0


def test_illegal_config_is_rejected():
    p = Conv2dGw8Params(n=1, c=64, h=8, w=16)
    with pytest.raises(AssertionError):
        conv2d_gw8_kernel_factory.get_kernel_spec(p, Conv2dGw8Config(groups=16, split=4), ATTR)
    with pytest.raises(ValueError):
        conv2d_gw8_kernel_factory.get_kernel_spec(p, Conv2dGw8Config(variant="nope"), ATTR)


def test_overlay_cache_semantics():
    """A non-empty overlay must contain the key (reference: kernel_cache.py:62-68)."""
    import torch

    cache = KernelCache()
    p = Conv2dGw8Params(n=1, c=8, h=4, w=4)
    sentinel = object()
    cache.update_overlay({KernelKey(device_ordinal=0, params=p): sentinel})
    dev = torch.device("cuda", 0)
    assert cache.get(conv2d_gw8_kernel_factory, p, dev) is sentinel
    with pytest.raises(ValueError, match="overlay"):
        cache.get(conv2d_gw8_kernel_factory, Conv2dGw8Params(n=2, c=8, h=4, w=4), dev)
    cache.clear_overlay()


def test_params_logger_records_requests():
    import torch

    cache = KernelCache()
    p = Conv2dGw8Params(n=1, c=8, h=4, w=4)
    cache.update_overlay({KernelKey(device_ordinal=0, params=p): object()})
    assert not kernel_params_logging_is_enabled()
    with KernelParamsLogger() as logger:
        assert kernel_params_logging_is_enabled()
        cache.get(conv2d_gw8_kernel_factory, p, torch.device("cuda", 0), igrad=True)
    assert not kernel_params_logging_is_enabled()
    (rec,) = logger.get_logged_params()
    assert rec.params == p and rec.kernel_kwargs == (("igrad", True),)
    assert rec.key == KernelKey(device_ordinal=0, params=p)


def test_tuner_record_store(tmp_path, monkeypatch):
    monkeypatch.setenv("SPIO_TUNE_DB", str(tmp_path / "db.json"))
    t = Tuner()
    assert t.lookup(ATTR, "k__x") is None
    t._store(ATTR, "k__x", {"config": {"groups": 8}, "us": 12.5})
    assert Tuner().lookup(ATTR, "k__x")["us"] == 12.5
    assert device_key(ATTR) == "gfx950_256cu"
    assert json.load(open(tmp_path / "db.json"))["k__x"]["config"] == {"groups": 8}


def test_small_image_shapes_offer_mover_wave_configurations():
    """The whole-image kernel is offered with and without data-mover waves for the small-image
    shapes; for 3x3 filters both are among the first candidates (a sweep cut short sees both)."""
    for shape in ("128n_384c_14h_14w_1py_1px_3r_3s_b", "256n_256c_14h_14w_3py_3px_7r_7s_nb"):
        params = Conv2dGw8Params.decode(shape)
        configs = conv2d_gw8_kernel_factory.configs(params, ATTR)
        image = [c for c in configs if c.variant == "image"]
        assert any(c.movers for c in image) and any(not c.movers for c in image)
        if params.r == 3:  # where moving a block takes longer than multiplying it
            assert {bool(c.movers) for c in configs[:4] if c.variant == "image"} == {False, True}
    # illegal: mover waves with single buffers, or more waves than a workgroup holds
    params = Conv2dGw8Params.decode("128n_384c_14h_14w_1py_1px_3r_3s_b")
    for bad in (Conv2dGw8Config(groups=8, block_p=14, variant="image", prefetch=1, movers=4, block_n_iters=2),
                Conv2dGw8Config(groups=8, block_p=14, variant="image", prefetch=2, movers=12, block_n_iters=2)):
        with pytest.raises(AssertionError):
            conv2d_gw8_kernel_factory.get_kernel_spec(params, bad, ATTR)


def test_layernorm_lane_choices():
    """Lanes per pixel: one unit per lane by default; where C/8 is not a power of two also the
    largest power of two dividing it, both among the first candidates."""
    from spio_amd.kernels import LayerNorm2dParams, layernorm_2d_kernel_factory

    expected = {96: 4, 192: 8, 384: 16, 768: 32, 64: None, 40: None, 2048: None}
    for c, exact in expected.items():
        params = LayerNorm2dParams(n=2, c=c, h=3, w=5)
        configs = layernorm_2d_kernel_factory.configs(params, ATTR)
        assert len(set(configs)) == len(configs)
        lanes = {cfg.lanes for cfg in configs}
        assert lanes == ({0, exact} if exact else {0})
        if exact:
            assert {cfg.lanes for cfg in configs[:2]} == {0, exact}
        for cfg in configs:
            spec = layernorm_2d_kernel_factory.get_kernel_spec(params, cfg, ATTR)
            lpp = spec.defines["SPIO_LN_LPP"]
            upl = -(-(c // 8) // lpp)
            assert lpp & (lpp - 1) == 0 and lpp * upl >= c // 8 and cfg.unroll * upl <= 8


def test_layernorm_eps_encodes_to_identifier_characters_and_round_trips():
    """The encoded parameters become part of the kernel's extern "C" symbol: every eps must give
    identifier characters only, decode back to the same value, and compile."""
    import re

    from spio_amd.kernels import LayerNorm2dParams, layernorm_2d_bwd_kernel_factory, layernorm_2d_kernel_factory

    assert LayerNorm2dParams(n=2, c=96, h=7, w=7).encode() == "2n_96c_7h_7w_1em06eps_wb"  # recorded names
    for eps in (1e-3, 1e-4, 0.1, 1.5e-5, 1e-12, 1e-5, 1e-6, 1.0, 2.5, 1e20):
        params = LayerNorm2dParams(n=2, c=96, h=7, w=7, eps=eps, has_bias=False)
        name = params.encode()
        assert re.fullmatch(r"[A-Za-z0-9_]+", name), name
        assert LayerNorm2dParams.decode(name) == params
    for factory in (layernorm_2d_kernel_factory, layernorm_2d_bwd_kernel_factory):
        for eps in (1e-3, 1.0):
            params = LayerNorm2dParams(n=2, c=96, h=7, w=7, eps=eps)
            kernel = factory.make_kernel(params, factory.configs(params, ATTR)[0], ATTR)
            kernel.compile()
            assert kernel.code


def test_fused_backward_works_on_the_larger_of_input_and_output():
    """The fused backward kernel's grid and loads per thread follow the domain both tensors sit in:
    the input's size where the output is smaller, the output's where it is larger; with an even
    filter size the two are offset by half a pixel and the domain holds both."""
    from spio_amd.kernels import Conv2dGw8BgradConfig, bgrad_is_supported
    from spio_amd.kernels.conv2d_gw8_bgrad_kernel import bgrad_domain, bgrad_geometry

    cfg = Conv2dGw8BgradConfig(groups=4, block_h=7, block_n=1)
    same = Conv2dGw8Params(n=4, c=32, h=28, w=28, padding=1)
    small = Conv2dGw8Params(n=4, c=32, h=28, w=28, padding=0)  # 26 x 26 output
    large = Conv2dGw8Params(n=4, c=32, h=28, w=28, padding=(3, 1))  # 32 x 28 output
    assert bgrad_domain(same) == bgrad_domain(small) == (28, 28) and bgrad_domain(large) == (32, 28)
    assert bgrad_geometry(small, cfg) == bgrad_geometry(same, cfg)
    assert bgrad_geometry(large, cfg)["PBLKS"] == 5 and bgrad_geometry(large, cfg)["STEPS"] == 7 + 3
    even = Conv2dGw8Params(n=4, c=32, h=28, w=28, r=4, s=1, padding=(2, 0))  # 29 x 28 output
    assert bgrad_domain(even) == (29, 28) and bgrad_geometry(even, cfg)["STEPS"] == 7 + 1 + 3
    assert bgrad_domain(Conv2dGw8Params(n=4, c=32, h=28, w=28, r=4, s=4, padding=(0, 3))) == (28, 31)
    assert all(bgrad_is_supported(p) for p in (same, small, large, even))


def test_weight_gradient_image_placement_reads_the_right_pixels():
    """The staged-row layout of the weight-gradient kernel (images sharing halo columns, chunks
    that hold their own images), restated from its constants: for every grad_output pixel and
    column tap, the x cell the contraction reads is that image's own column, or a cell no image
    ever writes (zero) where the column lies in the padding."""
    from spio_amd.kernels.conv2d_gw8_wgrad_kernel import image_placement

    cases = [(14, 7, 3, (1, 2, 3, 4, 5, 6, 8)), (14, 3, 1, (2, 4, 8)), (7, 3, 1, (4, 7, 8)), (10, 3, 1, (3, 6)),
             (15, 5, 2, (2, 4)), (13, 6, 4, (2, 4)), (28, 3, 1, (1, 2)), (9, 5, 0, (3, 5)), (12, 4, 3, (2, 4))]
    packed_seen = False
    for w, s, px, counts in cases:
        params = Conv2dGw8Params(n=8, c=16, h=w, w=w, r=1, s=s, padding=(0, px))
        q_width = params.q
        for nb in counts:
            g = image_placement(params, nb)
            ip, ipc, kc, xcp = g["IP"], g["IPC"], g["KC"], g["XCP"]
            packed_seen |= bool(g["PACKED"])
            d_off = [(i // ipc) * 32 + (i % ipc) * ip for i in range(nb)]
            x_off = [(i // ipc) * xcp + (i % ipc) * ip for i in range(nb)]
            assert max(d_off) + q_width <= 32 * kc
            assert kc <= (((nb - 1) * (q_width + s - 1) + q_width) + 31) // 32  # never more chunks than before
            owner = {}  # x cell -> (image, column) of the data it holds
            for i in range(nb):
                for col in range(params.w):
                    cell = x_off[i] + col + px
                    assert cell not in owner and cell < g["FPX"]
                    owner[cell] = (i, col)
            for i in range(nb):
                for q in range(q_width):
                    pos = d_off[i] + q
                    chunk, local = divmod(pos, 32)
                    for tap in range(s):
                        cell = chunk * xcp + local + tap  # what the B fragment of this tap reads
                        col = q + tap - px
                        if 0 <= col < params.w:
                            assert owner.get(cell) == (i, col), (w, s, px, nb, i, q, tap)
                        else:
                            assert cell not in owner, (w, s, px, nb, i, q, tap)
    assert packed_seen


def test_counter_figures_in_profiles_were_measured_with_the_committed_kernel_sources():
    """bench.py reads roofline.traffic and mfma_util from profiles/*.md; every such line names the
    kernel source and the digest of the text it was measured with.  A kernel edited after its
    profile was taken would make bench.py report traffic_stale: the committed state has none."""
    import importlib.util
    import re

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    seen = 0
    for workload in ("target", "cfg1", "cfg2", "cfg3"):
        for kernel in ("fprop", "dgrad", "wgrad", "bgrad"):
            for kind in ("traffic_bytes", "mfma_util"):
                value, stale = bench.profile_figure(kind, workload, kernel)
                if value is None:
                    assert (workload, kernel) == ("cfg3", "bgrad")  # 7x7 has no fused backward kernel
                    continue
                assert stale is False, (kind, workload, kernel)
                seen += 1
    assert seen == 30
    # the model bench.py prices every kernel against: launch floor + bytes at the copy's marginal rate
    m = bench.stream_model(18.3, 102769664)
    assert abs(m["stream_model_us"] - (2.2 + 102769664 / 6.2e6)) < 0.01 and 0.9 < m["frac_of_stream_model"] < 1.1
    assert re.fullmatch(r"[0-9a-f]{12}", bench.source_digest("conv2d_gw8_mfma.hip"))


def test_weight_gradient_mfma_kernel_is_not_offered_past_its_32_bit_indices():
    """The MFMA weight-gradient kernel indexes its tensors in 16-byte units with 32-bit integers:
    up to 32 GiB per tensor.  Beyond that only the general kernel (64-bit arithmetic) is offered;
    the forward and fused backward kernels rebase their descriptors per image block and stay."""
    from spio_amd.hip.driver import DeviceAttributes
    from spio_amd.kernels import (
        Conv2dGw8Params,
        conv2d_gw8_bgrad_kernel_factory,
        conv2d_gw8_kernel_factory,
        conv2d_gw8_wgrad_kernel_factory,
    )

    attr = DeviceAttributes()
    fits = Conv2dGw8Params(n=11000, c=64, h=56, w=56)  # 4.4 GB per tensor
    past = Conv2dGw8Params(n=90000, c=64, h=56, w=56)  # 36 GB per tensor
    assert {c.variant for c in conv2d_gw8_wgrad_kernel_factory.configs(fits, attr)} >= {"mfma"}
    assert {c.variant for c in conv2d_gw8_wgrad_kernel_factory.configs(past, attr)} == {"direct"}
    assert conv2d_gw8_kernel_factory.configs(past, attr)[0].variant == "mfma"
    assert conv2d_gw8_bgrad_kernel_factory.configs(past, attr)
