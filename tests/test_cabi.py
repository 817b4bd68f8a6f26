"""The C-ABI library: it loads, exports exactly what include/spio_hip.h declares,
compiles with hipRTC without a GPU, and rejects bad arguments.  CPU only (no
kernel is launched)."""

import ctypes
import os
import re

import pytest

from spio_amd.build import LIB_PATH, build_native
from spio_amd.hip import driver

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spio_hip.h")


def _declared_symbols():
    text = open(HEADER, "r", encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spio_hip[a-z_]*|spio_hiprtc_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(LIB_PATH):
        build_native()
    lib = ctypes.CDLL(LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 18
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in spio_hip.h but not exported"
    # ... and the Python binding knows a signature for each of them.
    assert sorted(driver._SIGNATURES) == declared


def test_error_before_init_is_reported():
    lib = ctypes.CDLL(LIB_PATH)
    lib.spio_hip_last_error.restype = ctypes.c_char_p
    # A separate dlopen shares the library state; only check the message format
    # of an argument error, which needs no device.
    driver.init()
    rc = lib.spio_hip_module_load(None, None)
    assert rc == 4  # SPIO_HIP_ERR_ARGUMENT
    assert b"null" in lib.spio_hip_last_error()


def test_hiprtc_compiles_for_gfx950_without_gpu():
    src = 'extern "C" __global__ void k(float* o) { o[__builtin_amdgcn_workitem_id_x()] = SPIO_V; }'
    prog = driver.Program(src, "k.hip")
    prog.compile(["--offload-arch=gfx950", "-DSPIO_V=3.0f"])
    code = prog.code()
    assert code[:4] == b"\x7fELF" and len(code) > 1000
    assert driver.get_hiprtc_version()[0] >= 6


def test_compile_error_raises_value_error_with_log():
    prog = driver.Program('extern "C" __global__ void k(float* o) { o[0] = undefined_symbol; }', "bad.hip")
    with pytest.raises(ValueError) as e:
        prog.compile(["--offload-arch=gfx950"])
    assert "undefined_symbol" in str(e.value) and "bad.hip" in str(e.value)
    with pytest.raises(ValueError):
        driver.Program("int x;", "x.hip").code()  # not compiled


def test_in_memory_header():
    prog = driver.Program('#include "v.h"\nextern "C" __global__ void k(float* o) { o[0] = V; }', "k.hip",
                          headers={"v.h": "#define V 2.0f\n"})  # fmt: skip
    prog.compile(["--offload-arch=gfx950"])
    assert len(prog.code()) > 1000


def test_argument_marshalling_rules():
    """None -> null pointer, int -> 64-bit, float -> 32-bit, more than 16 args rejected
    (reference: spio/cuda/driver.pyx:171-199)."""
    params, values = driver.Function.marshal([None, 5, 2.5, -3])
    assert len(params) == 4
    # params[i] is the address of the argument's own 8-byte slot, read as the kernel reads it
    assert ctypes.c_void_p.from_address(params[0]).value is None
    assert ctypes.c_longlong.from_address(params[1]).value == 5
    assert ctypes.c_float.from_address(params[2]).value == 2.5
    assert ctypes.c_longlong.from_address(params[3]).value == -3
    assert params[1] - params[0] == 8 and params[0] == ctypes.addressof(values)
    with pytest.raises(ValueError, match="Unsupported"):
        driver.Function.marshal([True])
    with pytest.raises(ValueError, match="64-bit"):
        driver.Function.marshal([1 << 70])
    with pytest.raises(ValueError, match="Too many"):
        driver.Function.marshal([0] * 17)
    with pytest.raises(ValueError, match="Unsupported"):
        driver.Function.marshal(["text"])


def test_launch_rejects_bad_geometry_without_touching_the_gpu():
    fn = driver.Function(0, "none")
    with pytest.raises(ValueError, match="null function"):
        fn.launch((1, 1, 1), (64, 1, 1), [])
    fn = driver.Function(1234, "fake")  # never dereferenced: geometry is checked first
    with pytest.raises(ValueError, match="zero-sized"):
        fn.launch((0, 1, 1), (64, 1, 1), [])
    with pytest.raises(ValueError, match="exceeds 1024"):
        fn.launch((1, 1, 1), (2048, 1, 1), [])
