"""One shape-specialised GPU kernel: compile, load, launch.

Reference: spio/kernels/kernel.py:22-174.  The reference generates a C++
header of typed dimensions per kernel; here every constant is a `-D` macro
(`KernelSpec.defines`) and the source is one of the HIP files in csrc/.
"""

from dataclasses import dataclass, field
from typing import Dict, Optional

import torch

from ..compiler.compile_kernel import compile_kernel, load_kernel
from ..compiler import flags
from ..hip.driver import launch_sequence_timed
from ..util.memory_format import check_channels_last
from .launch_params import LaunchParams


@dataclass
class KernelSpec:
    """Everything that specialises one kernel build and its launch.

    Attributes:
        defines: macro name -> value for the compilation.
        launch_params: grid, block and dynamic LDS bytes.
        source_file: HIP source inside csrc/.
        max_dynamic_lds: when set, the kernel's dynamic LDS limit is raised to it.
    """

    defines: Dict[str, object]
    launch_params: LaunchParams
    source_file: str
    max_dynamic_lds: Optional[int] = None
    notes: Dict[str, object] = field(default_factory=dict)
    # Two-stage kernels: the main kernel receives a workspace of `workspace_bytes` in place of
    # argument `workspace_arg`, then `<kernel name><epilogue_suffix>` runs with (that argument,
    # workspace, and the arguments listed in `epilogue_extra_args`) under `epilogue_launch_params`.
    workspace_bytes: int = 0
    epilogue_suffix: Optional[str] = None
    epilogue_launch_params: Optional[LaunchParams] = None
    workspace_arg: int = 0
    epilogue_extra_args: tuple = ()
    # True: the kernel (its last stage) stores the tensor at `workspace_arg` whole, so the caller
    # need not zero it; False: the kernel adds into it
    overwrites_output: bool = False



class LaunchTimer:
    """Times every Kernel.launch made while it is active, with HIP events on the launch stream.

        with LaunchTimer() as timer:
            model(x)
        timer.averages(skip=2)   # {kernel: average microseconds, first 2 launches left out}

    This is how kernels are timed in situ, inside a model with the cache state the model
    produces (the reference reads the same from torch.profiler,
    scripts/profile_block.py:646-701).
    """

    active = None

    def __init__(self):
        self.events = {}

    def __enter__(self):
        LaunchTimer.active = self
        self.events = {}
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        LaunchTimer.active = None
        return False

    def averages(self, skip: int = 0):
        """Average microseconds per launch of each kernel seen (after the first `skip`)."""
        torch.cuda.synchronize()
        out = {}
        for kernel, pairs in self.events.items():
            pairs = pairs[skip:] or pairs
            out[kernel] = 1e3 * sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)
        return out


class Kernel:
    """A compiled kernel bound to one device.  Made by KernelFactory.make_kernel."""

    def __init__(self, kernel_name, kernel_spec: KernelSpec, params=None, config=None,
                 args_checker=check_channels_last):  # fmt: skip
        self.kernel_name = kernel_name
        self.kernel_spec = kernel_spec
        self.params = params
        self.config = config
        self.args_checker = args_checker
        self.code: Optional[bytes] = None
        self.module = None
        self.function = None
        self.epilogue_function = None
        self.device_ordinal: Optional[int] = None

    @property
    def kernel_source_file(self) -> str:
        return self.kernel_spec.source_file

    @property
    def defines(self) -> Dict[str, object]:
        d = dict(self.kernel_spec.defines)
        d["SPIO_KERNEL_NAME"] = self.kernel_name
        return d

    def compile(self):
        """JIT-compile the specialised source to a code object."""
        self.code = compile_kernel(
            self.kernel_source_file, self.defines,
            debug=flags.debug.get(), lineinfo=flags.lineinfo.get(),
        )  # fmt: skip

    def load(self, device_ordinal: int = 0, clear_code: bool = True):
        """Load the code object on a device and resolve the kernel symbol."""
        if self.code is None:
            raise ValueError(f"Kernel {self.kernel_name} has not been compiled")
        self.module, self.function = load_kernel(self.kernel_name, self.code, device_ordinal)
        self.device_ordinal = device_ordinal
        if self.kernel_spec.epilogue_suffix:
            self.epilogue_function = self.module.get_function(
                self.kernel_name + self.kernel_spec.epilogue_suffix
            )
        if self.kernel_spec.max_dynamic_lds:
            self.function.set_max_dynamic_lds(self.kernel_spec.max_dynamic_lds)
        if clear_code:
            self.code = None

    def unload(self):
        """Drop the module; load() may be called again if the code was kept."""
        if self.module is not None:
            self.module.unload()
            self.module = None
        self.function = None
        self.epilogue_function = None

    def _prepare(self, args):
        """Check the arguments and return the device they live on."""
        if self.function is None:
            raise ValueError("kernel is not loaded")
        if self.args_checker is not None:
            self.args_checker(args)
        device = None
        for a in args:
            if isinstance(a, torch.Tensor) and a.numel() > 0:
                if device is None:
                    device = a.device
                elif a.device != device:
                    raise AssertionError("Not all tensor arguments are on the same device")
        if device is None or device.type != "cuda":
            raise ValueError("kernel arguments must be GPU tensors")
        return device

    def launch(self, *args, static_workspace: bool = False):
        """Asynchronous launch on torch's current stream of the arguments' device.

        `static_workspace=True` makes a two-stage kernel take its workspace from the native
        library's fixed device array instead of torch's allocator (for callers that must not
        allocate); it raises when the kernel needs more than that array holds, and launches that
        overlap on one GPU must not both use it.
        """
        try:
            device = self._prepare(args)
            spec = self.kernel_spec
            lp = spec.launch_params
            stream = torch.cuda.current_stream(device).cuda_stream
            timer = LaunchTimer.active
            if timer is not None:
                start = torch.cuda.Event(enable_timing=True)
                stop = torch.cuda.Event(enable_timing=True)
                timer.events.setdefault(self, []).append((start, stop))
                start.record()
            if self.epilogue_function is None:
                self.function.launch(lp.grid, lp.block, args, lp.shared_mem_bytes, stream)
            elif static_workspace:
                ep = spec.epilogue_launch_params
                nbytes = spec.workspace_bytes
                wa = spec.workspace_arg
                self.function.launch_scratch(lp.grid, lp.block, self._stage_args(args, None)[0], wa, nbytes,
                                             lp.shared_mem_bytes, stream)  # fmt: skip
                self.epilogue_function.launch_scratch(ep.grid, ep.block, self._stage_args(args, None)[1], 1, nbytes,
                                                      ep.shared_mem_bytes, stream)  # fmt: skip
            else:
                workspace = self._workspace(device)
                main_args, epilogue_args = self._stage_args(args, workspace)
                self.function.launch(lp.grid, lp.block, main_args, lp.shared_mem_bytes, stream)
                ep = spec.epilogue_launch_params
                self.epilogue_function.launch(ep.grid, ep.block, epilogue_args, ep.shared_mem_bytes, stream)
            if timer is not None:
                stop.record()
        except Exception as e:
            raise ValueError(f"Error in kernel {self}") from e

    def _stage_args(self, args, workspace):
        """Arguments of the two stages of a two-stage kernel: the main stage gets the workspace in
        place of argument `workspace_arg`, the second stage that argument, the workspace and the
        listed extra arguments (missing trailing ones, e.g. an absent grad_bias, become None)."""
        spec = self.kernel_spec
        wa = spec.workspace_arg
        args = tuple(args)
        main = args[:wa] + (workspace,) + args[wa + 1:]
        extra = tuple(args[i] if i < len(args) else None for i in spec.epilogue_extra_args)
        return main, (args[wa], workspace) + extra

    def _workspace(self, device) -> torch.Tensor:
        """Scratch for the partial results of a two-stage kernel (from torch's caching allocator)."""
        return torch.empty(self.kernel_spec.workspace_bytes, dtype=torch.uint8, device=device)

    def time(self, arg_sets, warmup: int = 3, iters: int = 20) -> float:
        """Average milliseconds per call (all stages), HIP events on torch's current stream."""
        device = None
        prepared = []
        for args in arg_sets:
            device = self._prepare(args)
            prepared.append(list(args))
        spec = self.kernel_spec
        lp = spec.launch_params
        stream = torch.cuda.current_stream(device).cuda_stream
        if self.epilogue_function is None:
            return self.function.launch_timed(
                lp.grid, lp.block, prepared, lp.shared_mem_bytes, stream, warmup, iters
            )
        ep = spec.epilogue_launch_params
        sets = []
        for kargs in prepared:
            ws = self._workspace(device)
            main_args, epilogue_args = self._stage_args(kargs, ws)
            sets.append([
                (self.function, lp.grid, lp.block, lp.shared_mem_bytes, list(main_args)),
                (self.epilogue_function, ep.grid, ep.block, ep.shared_mem_bytes, list(epilogue_args)),
            ])  # fmt: skip
        return launch_sequence_timed(sets, stream, warmup, iters)

    def __call__(self, *args):
        self.launch(*args)

    def __repr__(self) -> str:
        return f"{self.kernel_name} {self.config}"


def get_full_kernel_name(kernel_name: str, params) -> str:
    """`<kernel>__<params.encode()>` (reference: kernel.py:160-163)."""
    return f"{kernel_name}__{params.encode()}"
