"""Python side of the C ABI in include/spio_hip.h.

Mirrors the objects of the reference's driver layer: `Module` / `Function`
(spio/cuda/driver.pyx:126-242), `DeviceAttributes` / `get_device_attributes`
(:98-108, 360-369) and the run-time compiler `Program`
(spio/cuda/nvrtc_ctypes.py:152-217).  Failures raise `HipError`, a ValueError
like the reference's driver errors (driver.pyx:118-123).
"""

import ctypes
import os
import struct
import threading
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

from ..build import LIB_PATH, build_native


class HipError(ValueError):
    """An error reported by libspio_hip.so (HIP, hipRTC or argument checks)."""


class _DeviceAttrsStruct(ctypes.Structure):
    _fields_ = [
        ("compute_unit_count", ctypes.c_int),
        ("l2_cache_bytes", ctypes.c_int),
        ("max_lds_bytes_per_block", ctypes.c_int),
        ("wavefront_size", ctypes.c_int),
        ("clock_khz", ctypes.c_int),
        ("memory_clock_khz", ctypes.c_int),
        ("memory_bus_width_bits", ctypes.c_int),
        ("max_threads_per_block", ctypes.c_int),
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 64),
    ]


class _LaunchDesc(ctypes.Structure):
    _fields_ = [
        ("function", ctypes.c_void_p),
        ("grid", ctypes.c_uint * 3),
        ("block", ctypes.c_uint * 3),
        ("dynamic_lds_bytes", ctypes.c_uint),
        ("num_params", ctypes.c_int),
        ("params", ctypes.POINTER(ctypes.c_void_p)),
    ]


@dataclass(frozen=True)
class DeviceAttributes:
    """Static properties of one GPU.

    `multiprocessor_count` keeps the reference's field name
    (driver.pyx:98-108) for the compute-unit count.
    """

    multiprocessor_count: int = 256
    l2_cache_size: int = 4 * 1024 * 1024
    name: str = "AMD Instinct MI355X"
    arch: str = "gfx950"
    max_shared_memory_per_block: int = 160 * 1024
    wavefront_size: int = 64
    clock_khz: int = 2400000
    memory_clock_khz: int = 2000000
    memory_bus_width_bits: int = 8192
    max_threads_per_block: int = 1024


# Exported symbols and their ctypes signatures; also used by the tests that
# check the library against the header.
_vp = ctypes.c_void_p
_F32_BITS = struct.Struct("<f")  # a float argument travels as its IEEE-754 single bits
_F32 = struct.Struct("<I")
_SIGNATURES = {
    "spio_hip_init": ([ctypes.c_char_p, ctypes.c_char_p], ctypes.c_int),
    "spio_hip_last_error": ([], ctypes.c_char_p),
    "spio_hip_free": ([_vp], None),
    "spio_hip_compile": (
        [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
         ctypes.POINTER(ctypes.c_char_p), ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
         ctypes.POINTER(_vp), ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(_vp)],
        ctypes.c_int,
    ),
    "spio_hip_module_load": ([_vp, ctypes.POINTER(_vp)], ctypes.c_int),
    "spio_hip_module_unload": ([_vp], ctypes.c_int),
    "spio_hip_get_function": ([_vp, ctypes.c_char_p, ctypes.POINTER(_vp)], ctypes.c_int),
    "spio_hip_func_set_max_dynamic_lds": ([_vp, ctypes.c_int], ctypes.c_int),
    "spio_hip_launch": (
        [_vp] + [ctypes.c_uint] * 7 + [_vp, ctypes.POINTER(_vp), ctypes.c_int],
        ctypes.c_int,
    ),
    "spio_hip_launch_scratch": (
        [_vp] + [ctypes.c_uint] * 7 + [_vp, ctypes.POINTER(_vp), ctypes.c_int, ctypes.c_int, ctypes.c_size_t],
        ctypes.c_int,
    ),
    "spio_hip_launch_timed": (
        [_vp] + [ctypes.c_uint] * 7
        + [_vp, ctypes.POINTER(ctypes.POINTER(_vp)), ctypes.c_int, ctypes.c_int, ctypes.c_int,
           ctypes.c_int, ctypes.POINTER(ctypes.c_float)],
        ctypes.c_int,
    ),
    "spio_hip_launch_sequence_timed": (
        [ctypes.POINTER(_LaunchDesc), ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int,
         ctypes.POINTER(ctypes.c_float)],
        ctypes.c_int,
    ),
    "spio_hip_zero_fill_async": ([_vp, ctypes.c_size_t, _vp], ctypes.c_int),
    "spio_hip_device_count": ([ctypes.POINTER(ctypes.c_int)], ctypes.c_int),
    "spio_hip_device_attrs": ([ctypes.c_int, ctypes.POINTER(_DeviceAttrsStruct)], ctypes.c_int),
    "spio_hip_set_device": ([ctypes.c_int], ctypes.c_int),
    "spio_hip_synchronize": ([], ctypes.c_int),
    "spio_hip_stream_synchronize": ([_vp], ctypes.c_int),
    "spio_hip_driver_version": ([ctypes.POINTER(ctypes.c_int)], ctypes.c_int),
    "spio_hip_runtime_version": ([ctypes.POINTER(ctypes.c_int)], ctypes.c_int),
    "spio_hiprtc_version": ([ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)], ctypes.c_int),
}  # fmt: skip

# Size of the library's static device workspace (SPIO_HIP_SCRATCH_BYTES in spio_hip.h).
SCRATCH_BYTES = 32 * 1024 * 1024

_lib = None
_lib_lock = threading.Lock()
_initialized = False


def library_path() -> str:
    """Path of the native library this binding loads."""
    return LIB_PATH


def _load_library():
    """dlopen libspio_hip.so (building it when it has not been built yet)."""
    global _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            build_native(force=True)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
        return _lib


def _check(rc: int):
    if rc != 0:
        msg = _lib.spio_hip_last_error()
        raise HipError(f"{msg.decode(errors='replace') if msg else 'unknown error'} [code {rc}]")


def loaded_runtime_libraries() -> Dict[str, str]:
    """Paths of the HIP runtime / hipRTC copies already mapped in this process."""
    found = {}
    try:
        with open("/proc/self/maps", "r", encoding="utf-8") as f:
            for line in f:
                path = line.rsplit(" ", 1)[-1].strip()
                base = os.path.basename(path)
                if base.startswith("libamdhip64.so") and "hip" not in found:
                    found["hip"] = path
                elif base.startswith("libhiprtc.so") and "hiprtc" not in found:
                    found["hiprtc"] = path
    except OSError:
        pass
    return found


def _torch_lib_dir() -> Optional[str]:
    try:
        import torch  # pylint: disable=import-outside-toplevel

        return os.path.join(os.path.dirname(torch.__file__), "lib")
    except ImportError:
        return None


def init():
    """Bind the HIP runtime and hipRTC (idempotent).

    Prefers the libraries PyTorch already mapped, then the ones it ships, so
    that this layer and torch share one runtime (one primary context, the
    same streams and allocations); falls back to the system ROCm install.
    """
    global _initialized
    lib = _load_library()
    if _initialized:
        return
    mapped = loaded_runtime_libraries()
    tdir = _torch_lib_dir()
    hip_path = mapped.get("hip")
    rtc_path = mapped.get("hiprtc")
    if hip_path is None and tdir and os.path.exists(os.path.join(tdir, "libamdhip64.so")):
        hip_path = os.path.join(tdir, "libamdhip64.so")
    if rtc_path is None and hip_path is not None:
        cand = os.path.join(os.path.dirname(hip_path), "libhiprtc.so")
        if os.path.exists(cand):
            rtc_path = cand
    _check(
        lib.spio_hip_init(
            hip_path.encode() if hip_path else None, rtc_path.encode() if rtc_path else None
        )
    )
    _initialized = True


def is_initialized() -> bool:
    """Whether init() has bound the runtime."""
    return _initialized


class Program:
    """One translation unit compiled at run time with hipRTC.

    Same shape as the reference's NVRTC `Program`
    (spio/cuda/nvrtc_ctypes.py:152-217): construct with source text and
    in-memory headers, `compile(options)`, then read `code()` and `log()`.
    """

    def __init__(self, source: str, name: str, headers: Optional[Dict[str, str]] = None):
        self.source = source
        self.name = name
        self.headers = dict(headers or {})
        self._code: Optional[bytes] = None
        self._log: str = ""

    def compile(self, options: Sequence[str] = ()):
        """Compile to a code object; raises HipError with the compiler log."""
        init()
        names = list(self.headers.keys())
        n = len(names)
        hsrc = (ctypes.c_char_p * max(n, 1))(*[self.headers[k].encode() for k in names])
        hname = (ctypes.c_char_p * max(n, 1))(*[k.encode() for k in names])
        opts = [o.encode() for o in options]
        copts = (ctypes.c_char_p * max(len(opts), 1))(*opts)
        code = _vp()
        size = ctypes.c_size_t()
        log = _vp()
        rc = _lib.spio_hip_compile(
            self.source.encode(), self.name.encode(), n, hsrc, hname, len(opts), copts,
            ctypes.byref(code), ctypes.byref(size), ctypes.byref(log),
        )  # fmt: skip
        if log.value:
            self._log = ctypes.string_at(log.value).decode(errors="replace")
            _lib.spio_hip_free(log)
        if rc == 0:
            self._code = ctypes.string_at(code.value, size.value)
            _lib.spio_hip_free(code)
        _check(rc)

    def code(self) -> bytes:
        """The compiled code object."""
        if self._code is None:
            raise HipError("program has not been compiled")
        return self._code

    def log(self) -> str:
        """Compiler diagnostics of the last compile()."""
        return self._log


class Function:
    """A kernel inside a loaded module (reference: driver.pyx:126-208)."""

    MAX_ARGS = 16

    def __init__(self, handle: int, name: str):
        self._handle = handle
        self.name = name

    @property
    def handle(self) -> int:
        """Opaque function handle."""
        return self._handle

    def set_max_dynamic_lds(self, nbytes: int):
        """Raise the kernel's dynamic LDS limit."""
        _check(_lib.spio_hip_func_set_max_dynamic_lds(self._handle, int(nbytes)))

    @staticmethod
    def marshal(args) -> Tuple[object, object]:
        """Convert launch arguments to the `params` array of the C ABI.

        Follows the reference's conventions (driver.pyx:181-199): tensors pass
        their device pointer, None a null pointer, int a 64-bit integer, float
        a 32-bit float.  Every value sits in its own 8-byte slot of one array
        (a 32-bit float in the low bytes of its slot) and `params[i]` is the
        address of slot i.  Returns `params` and the slot array, which must be
        kept alive until the launch call returns.
        """
        n = len(args)
        if n > Function.MAX_ARGS:
            raise ValueError(f"Too many kernel arguments: {n} > {Function.MAX_ARGS}")
        slots = []
        for a in args:
            if a is None:
                slots.append(0)
            elif hasattr(a, "data_ptr"):
                slots.append(a.data_ptr())
            elif isinstance(a, bool):
                raise ValueError(f"Unsupported kernel argument type: {type(a)}")
            elif isinstance(a, int):
                if not -(1 << 63) <= a < (1 << 64):
                    raise ValueError(f"Integer kernel argument out of 64-bit range: {a}")
                slots.append(a & 0xFFFFFFFFFFFFFFFF)
            elif isinstance(a, float):
                slots.append(_F32.unpack(_F32_BITS.pack(a))[0])
            else:
                raise ValueError(f"Unsupported kernel argument type: {type(a)}")
        values = (ctypes.c_uint64 * max(n, 1))(*slots)
        base = ctypes.addressof(values)
        params = (_vp * max(n, 1))(*range(base, base + 8 * max(n, 1), 8))
        return params, values

    def launch(self, grid, block, args, shared_mem_bytes: int = 0, stream: int = 0):
        """Asynchronous launch on `stream` (an integer hipStream_t, 0 = null)."""
        params, _values = self.marshal(args)
        rc = _lib.spio_hip_launch(
            self._handle, grid[0], grid[1], grid[2], block[0], block[1], block[2],
            shared_mem_bytes, stream or None, params, len(args),
        )  # fmt: skip
        if rc:
            _check(rc)

    def launch_scratch(self, grid, block, args, scratch_param: int, scratch_bytes: int,
                       shared_mem_bytes: int = 0, stream: int = 0):  # fmt: skip
        """Launch with the library's static device workspace as argument `scratch_param`.

        Nothing is allocated; `args[scratch_param]` is ignored (pass None).  All calls on one
        GPU share the workspace, so launches that overlap on one GPU must not both use it.
        """
        params, _values = self.marshal(args)
        rc = _lib.spio_hip_launch_scratch(
            self._handle, grid[0], grid[1], grid[2], block[0], block[1], block[2],
            shared_mem_bytes, stream or None, params, len(args), int(scratch_param), int(scratch_bytes),
        )  # fmt: skip
        if rc:
            _check(rc)

    def launch_timed(
        self, grid, block, arg_sets: List[Sequence], shared_mem_bytes: int = 0, stream: int = 0,
        warmup: int = 3, iters: int = 20,
    ) -> float:  # fmt: skip
        """Average milliseconds per launch over `iters` launches.

        The launches run back to back between two HIP events on `stream`,
        cycling through `arg_sets`, after `warmup` untimed launches.
        """
        marshalled = [self.marshal(a) for a in arg_sets]
        nargs = len(arg_sets[0])
        sets = (ctypes.POINTER(_vp) * len(marshalled))(
            *[ctypes.cast(m[0], ctypes.POINTER(_vp)) for m in marshalled]
        )
        ms = ctypes.c_float()
        _check(
            _lib.spio_hip_launch_timed(
                self._handle, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                int(shared_mem_bytes), stream or None, sets, len(marshalled), nargs,
                int(warmup), int(iters), ctypes.byref(ms),
            )  # fmt: skip
        )
        return ms.value / iters


def launch_sequence_timed(launch_sets, stream: int = 0, warmup: int = 3, iters: int = 20) -> float:
    """Average milliseconds per iteration of a multi-kernel sequence.

    `launch_sets` is a list of argument sets; each set is a list of stages
    `(function, grid, block, shared_mem_bytes, args)` launched in order.
    Iterations cycle through the sets.
    """
    init()
    stages = len(launch_sets[0])
    descs = (_LaunchDesc * (stages * len(launch_sets)))()
    keep = []
    i = 0
    for launch_set in launch_sets:
        assert len(launch_set) == stages
        for function, grid, block, lds, args in launch_set:
            arr, storage = Function.marshal(args)
            keep.append((arr, storage))
            d = descs[i]
            d.function = function.handle
            d.grid = (ctypes.c_uint * 3)(*grid)
            d.block = (ctypes.c_uint * 3)(*block)
            d.dynamic_lds_bytes = int(lds)
            d.num_params = len(storage)
            d.params = ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p))
            i += 1
    ms = ctypes.c_float()
    _check(
        _lib.spio_hip_launch_sequence_timed(
            descs, stages, len(launch_sets), stream or None, int(warmup), int(iters), ctypes.byref(ms)
        )
    )
    return ms.value / iters


class Module:
    """A loaded code object (reference: driver.pyx:210-242)."""

    def __init__(self):
        self._handle = None

    def load_data(self, code: bytes):
        """Load a code object produced by Program.compile()."""
        init()
        if self._handle is not None:
            self.unload()
        self._code_ref = code
        handle = _vp()
        _check(_lib.spio_hip_module_load(code, ctypes.byref(handle)))
        self._handle = handle.value
        return self

    def get_function(self, name: str) -> Function:
        """Look up a kernel by name."""
        if self._handle is None:
            raise HipError("module is not loaded")
        fn = _vp()
        _check(_lib.spio_hip_get_function(self._handle, name.encode(), ctypes.byref(fn)))
        return Function(fn.value, name)

    def unload(self):
        """Unload the module; its functions become invalid."""
        if self._handle is not None:
            handle, self._handle = self._handle, None
            _check(_lib.spio_hip_module_unload(handle))

    def __del__(self):
        try:
            self.unload()
        except Exception:  # pylint: disable=broad-except
            pass


def get_device_attributes(device_ordinal: int = 0) -> DeviceAttributes:
    """Query the properties of a device."""
    init()
    s = _DeviceAttrsStruct()
    _check(_lib.spio_hip_device_attrs(int(device_ordinal), ctypes.byref(s)))
    return DeviceAttributes(
        multiprocessor_count=s.compute_unit_count,
        l2_cache_size=s.l2_cache_bytes,
        name=s.name.decode(errors="replace"),
        arch=s.arch.decode(errors="replace").split(":")[0] or "gfx950",
        max_shared_memory_per_block=s.max_lds_bytes_per_block,
        wavefront_size=s.wavefront_size,
        clock_khz=s.clock_khz,
        memory_clock_khz=s.memory_clock_khz,
        memory_bus_width_bits=s.memory_bus_width_bits,
        max_threads_per_block=s.max_threads_per_block,
    )


def _int_query(fn_name: str) -> int:
    init()
    v = ctypes.c_int()
    _check(getattr(_lib, fn_name)(ctypes.byref(v)))
    return v.value


def device_count() -> int:
    """Number of visible GPUs."""
    return _int_query("spio_hip_device_count")


def get_driver_version() -> int:
    """HIP driver version."""
    return _int_query("spio_hip_driver_version")


def get_runtime_version() -> int:
    """HIP runtime version."""
    return _int_query("spio_hip_runtime_version")


def get_hiprtc_version() -> Tuple[int, int]:
    """(major, minor) of hipRTC."""
    init()
    a, b = ctypes.c_int(), ctypes.c_int()
    _check(_lib.spio_hiprtc_version(ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def set_device(ordinal: int):
    """Make `ordinal` the current device of the calling thread."""
    init()
    _check(_lib.spio_hip_set_device(int(ordinal)))


def synchronize():
    """Block until the current device is idle."""
    init()
    _check(_lib.spio_hip_synchronize())


def stream_synchronize(stream: int = 0):
    """Block until `stream` is idle."""
    init()
    _check(_lib.spio_hip_stream_synchronize(stream or None))


def zero_fill_async(ptr: int, nbytes: int, stream: int = 0):
    """Zero `nbytes` of device memory asynchronously on `stream` with a fill kernel (any
    alignment, any size; safe to record under HIP graph capture)."""
    init()
    _check(_lib.spio_hip_zero_fill_async(ptr, nbytes, stream or None))
