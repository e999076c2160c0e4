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
        """From 5 to 8 rows and from 64 on.  With fewer rows the norm fused into the gate-up product
        costs little (few float rows to stage); from 5 on reading prepared bfloat16 rows beats staging
        float ones in every one of the product's many workgroups (a decode step at TinyLlama's sizes:
        1.020 -> 0.990 ms at 8 rows, no difference at 4, 0.918 -> 0.948 at one).  From 9 rows on the
        fused norm is out of reach and the choice is a norm kernel of its own: that is the faster way
        up to 63 rows, because every workgroup of the product has to add up the prepared parts (1.085
        against 1.072 ms at 16 rows, 1.269 against 1.252 at 32, 1.558 against 1.565 at 64).  Those are
        the weight-streaming kernel's figures: a wide gate-up product of 24 to 64 rows goes to the tiled
        kernel, which adds the parts up once a tile of 64 rows while its first operands are on their way
        and puts the rows' factors into its epilogue -- the norm's kernel goes (1.217 -> 1.178 ms at
        32 rows, 1.368 -> 1.322 at 64)."""
        if not self.interleaved:
            return False
        if n_rows <= ops.SKINNY_MAX_ROWS and ops.tiled_takes_prenormed(n_rows, *self.w_gu.shape):
            return True
        return 5 <= n_rows <= ops.NORMED_MAX_ROWS or (n_rows >= 64 and ops.streams_weights(n_rows, *self.w_gu.shape))

    def forward(self, h, ctx, residual) -> None:
        act = linear_swiglu(h, self.w_gu, self.interleaved)
        linear(act, self.w_down, accumulate_into=residual, ctx=ctx)


register_part("feedforward", "swiglu", SwiGLU)
