"""Replace eligible modules of a model by their spio_amd counterparts.

Reference: spio/transform/_transform.py:16-108.  `transform(model)` traces the
model with torch.fx, swaps every `nn.Conv2d` accepted by `Conv2dGw8.match` for a
`Conv2dGw8` that shares its parameters, and returns the recompiled GraphModule;
`scan_modules(model, *args)` runs the traced model once and reports the
`Conv2dGw8Params` of every module that would be replaced.
"""

from typing import List, Tuple

import torch
from torch import nn
from torch.fx import symbolic_trace

from ..layers import Conv2dGw8
from ..util.logger import logger_enabled

spio_modules_classes = [Conv2dGw8]


def _matching_class(module: nn.Module):
    for cls in spio_modules_classes:
        if cls.match(module):
            return cls
    return None


def count_replaceable(model: nn.Module) -> int:
    """Number of sub-modules `transform` would replace (no tracing needed)."""
    return sum(1 for m in model.modules() if _matching_class(m) is not None)


def _transform(model: nn.Module) -> Tuple[torch.fx.GraphModule, int]:
    traced = symbolic_trace(model)
    modules = dict(traced.named_modules())
    replaced = 0
    for node in list(traced.graph.nodes):
        if node.op != "call_module" or node.target not in modules:
            continue
        old = modules[node.target]
        cls = _matching_class(old)
        if cls is None:
            continue
        new = cls.from_torch_module(old)
        parent_name, _, leaf = node.target.rpartition(".")
        parent = modules[parent_name] if parent_name else traced
        setattr(parent, leaf, new)  # same target name: the graph node now calls the new module
        replaced += 1
        if logger_enabled:
            print(f"spio: replaced {type(old).__module__}.{type(old).__name__} '{node.target}' with {new}")
    traced.recompile()
    return traced, replaced


def transform(model: nn.Module) -> torch.fx.GraphModule:
    """The model with every eligible module replaced; parameters are shared, not copied."""
    return _transform(model)[0]


class _ScanInterpreter(torch.fx.Interpreter):
    def __init__(self, gm):
        super().__init__(gm)
        self._modules = dict(gm.named_modules())
        self.params_lst: List = []

    def call_module(self, target, args, kwargs):
        module = self._modules.get(target)
        cls = _matching_class(module) if module is not None else None
        if cls is not None:
            self.params_lst.append(cls.Params.from_torch_module(module, *args))
        return super().call_module(target, args, kwargs)


def scan_modules(model: nn.Module, *args) -> List:
    """Params of every module `transform` would replace, for the given example inputs."""
    interpreter = _ScanInterpreter(symbolic_trace(model))
    interpreter.run(*args)
    return interpreter.params_lst
