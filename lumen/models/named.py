"""Base of the model families whose parameters keep their checkpoint names.

A family that is served through a step function of its own (``lumen.serve.hybrid_runner``) holds
its tensors in one dictionary under the names the checkpoint uses (``l3.mix.q``), so loading is a
name-and-shape match and the serving weights are built from ``model.tensor(name)``.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn as nn


def _key(name: str) -> str:
    return name.replace(".", "/")        # a ParameterDict key may not contain dots


class NamedTensorModel(nn.Module):
    def __init__(self, config, shapes: Dict[str, tuple], dtype=torch.bfloat16, device=None):
        super().__init__()
        self.config = config
        self.dtype = dtype
        self.tensors = nn.ParameterDict()
        for name, shape in shapes.items():
            self.tensors[_key(name)] = nn.Parameter(
                torch.empty(shape, dtype=dtype, device=device), requires_grad=False)

    def tensor(self, name: str) -> torch.Tensor:
        return self.tensors[_key(name)]

    def tensor_names(self):
        return [k.replace("/", ".") for k in self.tensors.keys()]

    def has(self, name: str) -> bool:
        return _key(name) in self.tensors

    def replace_tensor(self, name: str, value: torch.Tensor) -> None:
        self.tensors[_key(name)] = nn.Parameter(value, requires_grad=False)
