"""Builds the native pieces of the package in-tree.

`build_native()` builds csrc/libspio_hip.so from csrc/spio_hip.cpp (host C++;
it binds the HIP runtime and hipRTC with dlopen) and the device sources
csrc/spio_hip_scratch.hip and csrc/spio_hip_fill.hip (hipcc, gfx950: the static
device workspace with the launch that uses it, and the zero-fill kernel; they
link the HIP runtime by its soname, so the copy a host framework has already
mapped is the one used).  hipcc cross-compiles, so this builds on machines
without a GPU.  Loading is another matter: because of the device translation
units the library has libamdhip64 as a link-time dependency and registers its
code objects when it is dlopen'ed, so every process that loads it, the
host-only tests and tools included, needs the HIP runtime library installed
(a GPU is not needed to load it).

`check_kernels()` compiles every HIP kernel source for gfx950 with hipcc for
a list of representative shape specialisations; at run time the same sources
are specialised per shape with hipRTC instead.
"""

import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_HERE, "csrc")
REPO_INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")
LIB_PATH = os.path.join(CSRC_DIR, "libspio_hip.so")
ROCM_HOME = os.environ.get("ROCM_PATH") or os.environ.get("ROCM_HOME") or "/opt/rocm"

# Device translation units of libspio_hip.so.
DEVICE_SOURCES = ["spio_hip_scratch.hip", "spio_hip_fill.hip"]

# hipcc flags shared by every device compilation of this package.
HIPCC_DEVICE_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _include_dir() -> str:
    """Directory holding spio_hip.h (repo layout or a copy inside csrc)."""
    if os.path.exists(os.path.join(REPO_INCLUDE_DIR, "spio_hip.h")):
        return REPO_INCLUDE_DIR
    return CSRC_DIR


def _run(cmd, what, verbose=False):
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")


def build_native(force: bool = True, verbose: bool = False) -> str:
    """Compile libspio_hip.so; returns its path."""
    host_src = os.path.join(CSRC_DIR, "spio_hip.cpp")
    dev_srcs = [os.path.join(CSRC_DIR, name) for name in DEVICE_SOURCES]
    deps = [host_src, *dev_srcs, os.path.join(CSRC_DIR, "spio_hip_internal.h"),
            os.path.join(_include_dir(), "spio_hip.h")]  # fmt: skip
    if not force and os.path.exists(LIB_PATH) and all(
        os.path.getmtime(LIB_PATH) >= os.path.getmtime(d) for d in deps
    ):
        return LIB_PATH
    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("no host C++ compiler found to build libspio_hip.so")
    hipcc = shutil.which("hipcc") or os.path.join(ROCM_HOME, "bin", "hipcc")
    includes = [f"-I{_include_dir()}", f"-I{CSRC_DIR}", f"-I{os.path.join(ROCM_HOME, 'include')}"]
    tag = f".tmp{os.getpid()}"
    host_obj = os.path.join(CSRC_DIR, f"spio_hip{tag}.o")
    dev_objs = [os.path.splitext(src)[0] + f"{tag}.o" for src in dev_srcs]
    tmp = LIB_PATH + tag
    try:
        _run([cxx, "-O2", "-std=c++17", "-fPIC", "-Wall", "-fvisibility-inlines-hidden", *includes,
              "-c", "-o", host_obj, host_src], "compiling spio_hip.cpp", verbose)  # fmt: skip
        for src, obj in zip(dev_srcs, dev_objs):
            _run([hipcc, *HIPCC_DEVICE_FLAGS, "-fPIC", *includes, "-c", "-o", obj, src],
                 f"compiling {os.path.basename(src)}", verbose)  # fmt: skip
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, host_obj, *dev_objs,
              "-ldl", "-lpthread"], "linking libspio_hip.so", verbose)  # fmt: skip
        os.replace(tmp, LIB_PATH)
    finally:
        for f in (host_obj, *dev_objs, tmp):
            if os.path.exists(f):
                os.remove(f)
    return LIB_PATH


def hipcc_compile_check(source_path: str, defines: dict, out_dir: str, tag: str) -> str:
    """Compile one kernel source to a gfx950 code object with hipcc."""
    hipcc = shutil.which("hipcc") or os.path.join(ROCM_HOME, "bin", "hipcc")
    out = os.path.join(out_dir, f"{tag}.co")
    cmd = [hipcc, "--genco", *HIPCC_DEVICE_FLAGS, f"-I{CSRC_DIR}"]
    cmd += [f"-D{k}={v}" for k, v in defines.items()]
    cmd += ["-o", out, source_path]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {tag}:\n{' '.join(cmd)}\n{proc.stderr}")
    return out


if __name__ == "__main__":
    print(build_native(verbose=True))
    sys.exit(0)
