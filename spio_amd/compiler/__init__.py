"""Run-time compilation of the HIP kernels with hipRTC."""

from .flags import lineinfo, debug, workers, code_cache_enabled
from .compile import compile_hip, hiprtc_options, GFX_ARCH
from .compile_kernel import compile_kernel, load_kernel, compile_and_load_kernel
from .compiler_pool import compile_kernels, compile_kernel_configs
