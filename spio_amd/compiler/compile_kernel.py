"""Compile and load one kernel from the package's csrc directory.

Reference: spio/compiler/compile_kernel.py:14-77 (`compile_kernel`,
`load_kernel`, `compile_and_load_kernel`).
"""

import functools
import os
from typing import Dict, Optional, Tuple

from ..build import CSRC_DIR
from ..hip.driver import Function, Module, set_device
from .compile import compile_hip, GFX_ARCH

# Headers that kernel sources may include; handed to hipRTC as in-memory files.
_HEADER_NAMES = ("spio_conv_common.h",)


@functools.lru_cache(maxsize=None)
def read_source(file_name: str) -> str:
    """Text of a file in csrc/."""
    with open(os.path.join(CSRC_DIR, file_name), "r", encoding="utf-8") as f:
        return f.read()


def kernel_headers() -> Dict[str, str]:
    """The in-memory header set for hipRTC."""
    return {name: read_source(name) for name in _HEADER_NAMES}


def compile_kernel(
    source_file_name: str,
    defines: Optional[Dict[str, object]] = None,
    arch: str = GFX_ARCH,
    debug: bool = False,
    lineinfo: bool = False,
) -> bytes:
    """Compile csrc/<source_file_name> with the given -D macros."""
    return compile_hip(
        read_source(source_file_name),
        source_file_name,
        headers=kernel_headers(),
        defines=defines,
        arch=arch,
        device_debug=debug,
        lineinfo=lineinfo,
    )


def load_kernel(kernel_name: str, code: bytes, device_ordinal: int = 0) -> Tuple[Module, Function]:
    """Load a code object on a device and look up its kernel."""
    set_device(device_ordinal)
    module = Module().load_data(code)
    return module, module.get_function(kernel_name)


def compile_and_load_kernel(
    kernel_name: str,
    source_file_name: str,
    defines: Optional[Dict[str, object]] = None,
    device_ordinal: int = 0,
    debug: bool = False,
    lineinfo: bool = False,
) -> Tuple[Module, Function]:
    """Compile then load; the kernel's symbol is `kernel_name`."""
    defines = dict(defines or {})
    defines.setdefault("SPIO_KERNEL_NAME", kernel_name)
    code = compile_kernel(source_file_name, defines, debug=debug, lineinfo=lineinfo)
    return load_kernel(kernel_name, code, device_ordinal)
