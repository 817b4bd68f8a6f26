"""On-device configuration sweep with recorded choices.

The reference predicts the best tile configuration with per-device XGBoost
models downloaded from its release page
(spio/kernels/performance_model_cache.py:102-124, 226-240, 432-479).  Here the
choice is measured: on the first request for a (kernel, params) pair every
legal configuration is compiled, timed on the device with HIP events over
rotating synthetic buffers, and the fastest one is recorded in a JSON file
keyed by device model (architecture + CU count) and full kernel name.  Later processes read the record
and compile only the winner.

Environment:
  SPIO_TUNE=0      never sweep; use the first (heuristically best) configuration
  SPIO_TUNE=1      sweep on a miss (default)
  SPIO_TUNE=force  sweep even when a record exists
  SPIO_TUNE_DB     path of the record file (default: <cache dir>/tune/<arch>_<CUs>cu.json)
  SPIO_TUNE_MAX_CONFIGS  how many configurations (the first ones of the ranked list) a sweep that
                   starts inside an operator call may try (default 8); `python -m spio_amd.tune`
                   and `tune_model` always try all of them

A sweep never starts while the current stream is being captured into a HIP graph (it allocates
and synchronises): the first configuration is used then, and nothing is recorded.

Before a winner is recorded its output on the synthetic arguments is compared with that of an
independent implementation (the direct kernel of the family where there is one, else the
candidate that differs most in tile geometry); a winner that disagrees is discarded.
"""

import dataclasses
import json
import os
import threading
import sys
import time
from typing import Any, Dict, List, Optional

from ..compiler.compiler_pool import compile_kernel_configs
from ..util.cache_dir import get_cache_dir
from ..util.logger import logger_enabled

_PACKAGE_RECORDS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuned")

# Rotate the timed launches over buffer sets totalling at least this many bytes
# so that the sweep ranks configurations by their HBM behaviour, not by hits in
# the 256 MB memory-side cache.
ROTATION_BYTES = 600 * 1024 * 1024
MAX_ROTATION_SETS = 8
DEFAULT_ON_MISS_CONFIGS = 8
FINALISTS = 6  # leaders of a sweep that are timed again before one is chosen


def _on_miss_limit() -> int:
    try:
        return max(1, int(os.environ.get("SPIO_TUNE_MAX_CONFIGS", DEFAULT_ON_MISS_CONFIGS)))
    except ValueError:
        return DEFAULT_ON_MISS_CONFIGS


def _stream_is_capturing() -> bool:
    try:
        import torch  # pylint: disable=import-outside-toplevel

        return bool(torch.cuda.is_current_stream_capturing())
    except Exception:  # pylint: disable=broad-except
        return False


def _outputs_agree(a, b) -> bool:
    """Loose agreement of two kernels' results on the same arguments (fp16 tensors: the
    operator's tolerance; fp32 sums: relative to the largest value)."""
    import torch  # pylint: disable=import-outside-toplevel

    for x, y in zip(a, b):
        if not (torch.isfinite(x).all() and torch.isfinite(y).all()):
            return False
        x32, y32 = x.float(), y.float()
        scale = float(y32.abs().max().clamp_min(1e-6))
        if x.dtype == torch.float16:
            ok = torch.allclose(x32, y32, rtol=4e-3, atol=2e-2 * max(1.0, scale / 16.0))
        else:
            ok = float((x32 - y32).abs().max()) <= 2e-3 * scale
        if not ok:
            return False
    return True


def _mode() -> str:
    return os.environ.get("SPIO_TUNE", "1").strip().lower()


def device_key(device_attr) -> str:
    """Identifies a device model in record file names: architecture and compute-unit count.

    The marketing name is not used: the runtime reports different strings for the same board
    depending on what is loaded in the process (a profiler, for one).
    """
    arch = "".join(ch if ch.isalnum() else "_" for ch in str(device_attr.arch).strip().lower())
    return f"{arch or 'unknown'}_{int(device_attr.multiprocessor_count)}cu"


def _device_file_name(device_attr) -> str:
    return device_key(device_attr) + ".json"


def config_to_dict(config) -> Dict[str, Any]:
    return dataclasses.asdict(config)


class Tuner:
    """Picks (and remembers) the fastest configuration of a kernel."""

    def __init__(self):
        self._lock = threading.RLock()
        self._records: Dict[str, Dict[str, Any]] = {}  # device file name -> records
        self.last_sweep: Optional[List[Dict[str, Any]]] = None

    # -- record storage -------------------------------------------------
    def _user_path(self, device_attr) -> str:
        override = os.environ.get("SPIO_TUNE_DB")
        if override:
            return override
        return os.path.join(get_cache_dir("tune"), _device_file_name(device_attr))

    def _load(self, device_attr) -> Dict[str, Any]:
        fname = _device_file_name(device_attr)
        recs = self._records.get(fname)
        if recs is not None:
            return recs
        recs = {}
        for path in (os.path.join(_PACKAGE_RECORDS, fname), self._user_path(device_attr)):
            try:
                with open(path, "r", encoding="utf-8") as f:
                    recs.update(json.load(f))
            except (OSError, ValueError):
                pass
        self._records[fname] = recs
        return recs

    def _store(self, device_attr, kernel_name: str, record: Dict[str, Any], path: Optional[str] = None):
        recs = self._load(device_attr)
        recs[kernel_name] = record
        path = path or self._user_path(device_attr)
        try:
            on_disk = {}
            try:
                with open(path, "r", encoding="utf-8") as f:
                    on_disk = json.load(f)
            except (OSError, ValueError):
                pass
            on_disk[kernel_name] = record
            tmp = f"{path}.{os.getpid()}.tmp"
            with open(tmp, "w", encoding="utf-8") as f:
                json.dump(on_disk, f, indent=1, sort_keys=True)
            os.replace(tmp, path)
        except OSError:
            pass

    def lookup(self, device_attr, kernel_name: str) -> Optional[Dict[str, Any]]:
        """The stored record for a kernel on a device, if any."""
        with self._lock:
            return self._load(device_attr).get(kernel_name)

    # -- selection ------------------------------------------------------
    def best_kernel(self, kernel_factory, params, ordinal, device_attr, **kernel_kwargs):
        """A compiled, loaded kernel using the best known configuration."""
        from .kernel_cache import compile_and_load_kernel  # circular at import time

        with self._lock:
            configs = list(kernel_factory.configs(params, device_attr, **kernel_kwargs))
            if not configs:
                raise ValueError(f"no kernel configuration supports {params}")
            name = kernel_factory.get_full_kernel_name(params, **kernel_kwargs)
            if all(getattr(c, "variant", "mfma") == "direct" for c in configs):
                # not an error, but a cliff the user should hear about: no MFMA tiling fits
                # (registers, LDS or the unrolled-step limit), the any-shape kernel runs
                print(f"spio: {name}: no MFMA configuration fits this shape; the any-shape kernel "
                      "is used and runs at a fraction of the MFMA kernels' throughput", file=sys.stderr)  # fmt: skip
            mode = _mode()
            record = None if mode == "force" else self.lookup(device_attr, name)
            if record is not None:
                try:
                    config = kernel_factory.config_cls(**record["config"])
                except TypeError:
                    config = None
                if config in configs:
                    return compile_and_load_kernel(
                        kernel_factory, params, config, ordinal, device_attr, **kernel_kwargs
                    )
            if mode in ("0", "false", "off", "no") or len(configs) == 1 or _stream_is_capturing():
                return compile_and_load_kernel(
                    kernel_factory, params, configs[0], ordinal, device_attr, **kernel_kwargs
                )
            # inside an operator call: only the best-ranked few, so that a model with many new
            # shapes does not stall (the last entry of a list is its any-shape kernel: keep it as
            # the independent implementation the winner is checked against)
            limit = _on_miss_limit()
            if len(configs) > limit + 1:
                configs = configs[:limit] + [configs[-1]]
            return self.sweep(kernel_factory, params, ordinal, device_attr, configs, **kernel_kwargs)

    def sweep(self, kernel_factory, params, ordinal, device_attr, configs=None, warmup=2,
              iters=8, record_path=None, **kernel_kwargs):  # fmt: skip
        """Time every configuration; record and return the fastest kernel (loaded)."""
        import torch  # pylint: disable=import-outside-toplevel

        if configs is None:
            configs = list(kernel_factory.configs(params, device_attr, **kernel_kwargs))
        name = kernel_factory.get_full_kernel_name(params, **kernel_kwargs)
        t0 = time.perf_counter()
        kernels = compile_kernel_configs(
            kernel_factory, params, configs=configs, device_attr=device_attr, **kernel_kwargs
        )
        device = torch.device("cuda", ordinal)
        first = kernel_factory.make_test_args(params, device, **kernel_kwargs)
        set_bytes = sum(a.numel() * a.element_size() for a in first if hasattr(a, "numel"))
        nsets = max(1, min(MAX_ROTATION_SETS, -(-ROTATION_BYTES // max(set_bytes, 1))))
        arg_sets = [first] + [
            kernel_factory.make_test_args(params, device, **kernel_kwargs) for _ in range(nsets - 1)
        ]
        results = []
        timed = []
        for kernel in kernels:
            try:
                kernel.load(device_ordinal=ordinal, clear_code=False)
                ms = kernel.time(arg_sets, warmup=warmup, iters=iters)
            except ValueError as e:
                results.append({"config": config_to_dict(kernel.config), "error": str(e)[:200]})
                kernel.unload()
                continue
            results.append({"config": config_to_dict(kernel.config), "us": ms * 1e3})
            timed.append((ms, kernel))
            kernel.unload()
        if not timed:
            raise ValueError(f"every configuration of {name} failed: {results}")
        timed.sort(key=lambda mk: mk[0])
        # The first pass is short; candidates within a few per cent of each other are ranked by
        # noise.  Time the leaders again, longer and several times, and order them by the median.
        finalists = [mk for mk in timed[:FINALISTS] if mk[0] <= 1.15 * timed[0][0]]
        if len(finalists) > 1:
            refined = []
            for _, kernel in finalists:
                kernel.load(device_ordinal=ordinal, clear_code=False)
                runs = sorted(kernel.time(arg_sets, warmup=2, iters=max(iters, 30)) for _ in range(5))
                kernel.unload()
                refined.append((runs[2], kernel))
                for r in results:
                    if r.get("config") == config_to_dict(kernel.config) and "us" in r:
                        r["us"] = runs[2] * 1e3
            refined.sort(key=lambda mk: mk[0])
            timed = refined + timed[len(finalists):]
        best = self._first_valid(kernel_factory, params, timed, first, ordinal, results)
        del arg_sets, first
        for _, kernel in timed:
            kernel.code = None  # loaded or discarded: the code objects are not needed any more
        record = {
            "config": config_to_dict(best[1].config),
            "us": best[0] * 1e3,
            "candidates": len(configs),
            "sweep": sorted((r for r in results if "us" in r), key=lambda r: r["us"])[:8],
        }
        self._store(device_attr, name, record, record_path)
        self.last_sweep = results
        if logger_enabled:
            print(
                f"spio: tuned {name}: {best[1].config} {best[0] * 1e3:.1f} us "
                f"({len(configs)} configs, {time.perf_counter() - t0:.1f} s)"
            )
        return best[1]


    # -- validation of a sweep's winner ------------------------------------
    @staticmethod
    def _run_outputs(kernel_factory, params, kernel, args, ordinal):
        """Run `kernel` once on copies of the synthetic arguments; returns its output tensors."""
        import torch  # pylint: disable=import-outside-toplevel

        # outputs come first in every kernel family here: (dst, ...), (dw, ...), (dx, dw, ...),
        # (sums, dx, ...); the gradient kernels of a layer with a bias take grad_bias as their
        # last argument
        family = kernel.kernel_name.split("__")[0]
        n_out = 2 if family.endswith(("bgrad", "_bwd")) else 1
        trailing_out = family.endswith(("wgrad", "bgrad")) and getattr(params, "has_bias", False)
        call = list(args)
        outs = []
        for i, a in enumerate(call):
            if not hasattr(a, "numel"):
                continue
            if i < n_out or (trailing_out and i == len(call) - 1):
                call[i] = torch.zeros_like(a)  # accumulated outputs start from zero
                outs.append(call[i])
        kernel.load(device_ordinal=ordinal, clear_code=False)
        try:
            kernel(*call)
            torch.cuda.synchronize()
        finally:
            kernel.unload()
        return outs

    def _first_valid(self, kernel_factory, params, timed, args, ordinal, results):
        """The fastest kernel whose result agrees with an independent implementation; loaded."""
        if len(timed) == 1:
            timed[0][1].load(device_ordinal=ordinal, clear_code=False)
            return timed[0]
        direct = [k for _, k in timed if getattr(k.config, "variant", "mfma") == "direct"]
        if direct:
            reference = direct[0]
        else:
            # no any-shape kernel in this family: the candidate furthest from the winner in tile
            # geometry (most differing configuration fields)
            w = config_to_dict(timed[0][1].config)
            reference = max((k for _, k in timed[1:]),
                            key=lambda k: sum(v != w.get(f) for f, v in config_to_dict(k.config).items()))
        try:
            expected = self._run_outputs(kernel_factory, params, reference, args, ordinal)
        except ValueError:
            timed[0][1].load(device_ordinal=ordinal, clear_code=False)
            return timed[0]
        for ms, kernel in timed:
            if kernel is reference:
                kernel.load(device_ordinal=ordinal, clear_code=False)
                return ms, kernel
            got = self._run_outputs(kernel_factory, params, kernel, args, ordinal)
            if _outputs_agree(got, expected):
                kernel.load(device_ordinal=ordinal, clear_code=False)
                return ms, kernel
            results.append({"config": config_to_dict(kernel.config), "rejected": "result differs from "
                            f"{reference.config}"})  # fmt: skip
            print(f"spio: sweep of {kernel.kernel_name}: configuration {kernel.config} disagrees with "
                  f"{reference.config} and was discarded")  # fmt: skip
        raise ValueError(f"no configuration of {timed[0][1].kernel_name} agrees with {reference.config}")


tuner = Tuner()
