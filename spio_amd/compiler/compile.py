"""Compile HIP source text to a gfx950 code object.

Reference: spio/compiler/compile.py:22-77 builds the NVRTC option list
(-arch, -G, -lineinfo, include paths) and raises ValueError carrying the
compiler log on failure.  Here the options go to hipRTC, every shape constant
is a -D macro, and compiled code objects are memoised on disk by a hash of
everything that determines them.
"""

import hashlib
import os
from typing import Dict, List, Optional

from ..hip.driver import Program, get_hiprtc_version
from ..util.cache_dir import get_cache_dir
from . import flags

GFX_ARCH = "gfx950"

# hipcc-side feature switch required for every device compilation here.
_FEATURE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hiprtc_options(
    defines: Optional[Dict[str, object]] = None,
    arch: str = GFX_ARCH,
    device_debug: bool = False,
    lineinfo: bool = False,
    extra: Optional[List[str]] = None,
) -> List[str]:
    """The option list for one compilation."""
    opts = [f"--offload-arch={arch}", "-std=c++17", "-O3", *_FEATURE_FLAGS]
    if device_debug:
        opts[2] = "-O0"
        opts.append("-g")
    elif lineinfo:
        opts.append("-gline-tables-only")
    for key, value in (defines or {}).items():
        if isinstance(value, bool):
            value = int(value)
        opts.append(f"-D{key}={value}" if value is not None else f"-D{key}")
    if extra:
        opts.extend(extra)
    return opts


def _cache_path(source: str, headers: Dict[str, str], options: List[str]) -> str:
    h = hashlib.sha256()
    h.update(repr(get_hiprtc_version()).encode())
    h.update(source.encode())
    for name in sorted(headers):
        h.update(name.encode())
        h.update(headers[name].encode())
    h.update("\0".join(options).encode())
    return os.path.join(get_cache_dir("code"), h.hexdigest() + ".co")


def compile_hip(
    source: str,
    name: str,
    headers: Optional[Dict[str, str]] = None,
    defines: Optional[Dict[str, object]] = None,
    arch: str = GFX_ARCH,
    device_debug: bool = False,
    lineinfo: bool = False,
    extra_options: Optional[List[str]] = None,
) -> bytes:
    """Compile `source` (with in-memory `headers`) and return the code object."""
    headers = dict(headers or {})
    options = hiprtc_options(defines, arch, device_debug, lineinfo, extra_options)
    use_cache = flags.code_cache_enabled.get()
    path = None
    if use_cache:
        try:
            path = _cache_path(source, headers, options)
            if os.path.exists(path):
                with open(path, "rb") as f:
                    data = f.read()
                if data:
                    return data
        except OSError:
            path = None
    program = Program(source, name, headers)
    program.compile(options)
    code = program.code()
    if path is not None:
        try:
            tmp = f"{path}.{os.getpid()}.tmp"
            with open(tmp, "wb") as f:
                f.write(code)
            os.replace(tmp, path)
        except OSError:
            pass
    return code
