"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear, linear_swiglu


class SwiGLU(Part):
    """x += (silu(h Wg^T) * (h Wu^T)) Wd^T with silu(g) = g / (1 + exp(-g)), no
    biases (reference: engine/src/model.cpp:579-603, engine/kernels/swiglu.cu:17-25)."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_gu = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": WeightSpec((i, h)), "up_proj.weight": WeightSpec((i, h)),
                "down_proj.weight": WeightSpec((h, i))}

    def bind(self, tensors, rt) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        # one product for gate and up: gate's rows, then up's
        self.w_gu = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, residual) -> None:
        act = linear_swiglu(h, self.w_gu)
        linear(act, self.w_down, accumulate_into=residual)


register_part("feedforward", "swiglu", SwiGLU)
