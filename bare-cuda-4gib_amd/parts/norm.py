"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, with eps on the mean square and
sum and rsqrt in float (reference: engine/kernels/rmsnorm.cu:16-41)."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..weights.loader import WeightSpec
from .base import Part, register_part


class RMSNorm(Part):
    category = "norm"
    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.size,), kind="vector", init="ones")}

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"]
        self.out_dtype = rt.act_dtype

    def fusable(self):
        """What a product needs to absorb this norm: (scale vector, eps)."""
        return self.weight, self.eps

    def forward(self, x: torch.Tensor, ctx=None, rows=None, n_rows=None) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.out_dtype, rows=rows, n_rows=n_rows)


register_part("norm", "rmsnorm", RMSNorm)
