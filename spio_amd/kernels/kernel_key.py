"""Cache keys (reference: spio/kernels/kernel_key.py:13-34)."""

from dataclasses import dataclass
from typing import Any, Tuple


@dataclass(frozen=True)
class KernelKey:
    """Key of a kernel in a KernelCache."""

    device_ordinal: int
    params: Any


@dataclass(frozen=True)
class KernelParams:
    """One kernel request captured by KernelParamsLogger."""

    kernel_cache: Any
    kernel_factory: Any
    params: Any
    device: Any
    kernel_kwargs: Tuple[Tuple[str, Any], ...]

    @property
    def key(self) -> KernelKey:
        """The key KernelCache.get files this request under: a device without an index means the
        current device, as it does there."""
        idx = self.device.index
        if idx is None:
            import torch  # pylint: disable=import-outside-toplevel

            idx = torch.cuda.current_device()
        return KernelKey(device_ordinal=idx, params=self.params)
