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
        i, h = self.intermediate_size, self.hidden_size
        # One product for gate and up.  For the matrix-core kernels (bfloat16, I a multiple of 8) the
        # rows go in blocks of 16 -- eight gate rows, then the eight up rows of the same outputs -- so
        # that one workgroup of the weight-streaming kernel holds both halves of its outputs;
        # otherwise gate's rows, then up's.
        self.interleaved = dt == torch.bfloat16 and i % 8 == 0
        if self.interleaved:
            self.w_gu = torch.stack([g.view(i // 8, 8, h), u.view(i // 8, 8, h)], dim=1).reshape(2 * i, h).contiguous()
        else:
            self.w_gu = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        self.w_gu = ops.StreamedWeight(self.w_gu)
        self.w_down = ops.StreamedWeight(tensors["down_proj.weight"])
        self.act_dtype = rt.act_dtype

    def wants_prepared_norm(self, n_rows: int) -> bool:
        """Whether the gate-up product, at this many rows, is better served by a norm that the product before
        prepared than by fusing the norm or running it: the weight's own plan says (ops.LinearPlan.wants_prepared)."""
        return self.interleaved and self.w_gu.plan.wants_prepared(n_rows, swiglu=True)

    def forward(self, h, ctx, residual) -> None:
        act = linear_swiglu(h, self.w_gu, self.interleaved)
        linear(act, self.w_down, accumulate_into=residual, ctx=ctx)


register_part("feedforward", "swiglu", SwiGLU)
