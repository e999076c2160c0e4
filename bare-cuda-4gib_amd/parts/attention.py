"""Causal softmax attention with grouped queries over the paged cache."""
from __future__ import annotations

import math
from typing import Dict

import torch

from ..cache.specs import PagedKV
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, build_part, register_part
from .linear import linear


class CausalAttention(Part):
    """q, k, v = h Wq^T, h Wk^T, h Wv^T (no biases); position encoding on q and
    k; k and v appended to the cache; scores = q.k / sqrt(head_dim) over the
    keys at or before the row's position (within ``window`` if it is not 0);
    query head h reads key/value head h // (num_heads / num_kv_heads); float
    softmax; output projection added to the residual stream.
    (Reference: engine/src/model.cpp:540-577, engine/kernels/attention_qk.cu:25-68.)"""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 window: int = 0, position=None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ConfigError(f"attention: {num_heads} heads cannot share {num_kv_heads} key/value heads")
        if window < 0:
            raise ConfigError(f"attention: window must not be negative, got {window}")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.num_kv_heads, self.head_dim, self.window = int(num_kv_heads), int(head_dim), int(window)
        self.position = build_part("position", position) if position is not None else None
        self.scale = 1.0 / math.sqrt(self.head_dim)
        self.w_qkv = self.w_o = None

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_spec(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def attention_tile_tokens(self) -> int:
        """Tokens per 16-row tile the matrix-core kernel wants the batch cut into."""
        return ops.attention_tile_tokens(self.num_heads, self.num_kv_heads)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        q, kv, h = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim, self.hidden_size
        return {"q_proj.weight": WeightSpec((q, h)), "k_proj.weight": WeightSpec((kv, h)),
                "v_proj.weight": WeightSpec((kv, h)), "o_proj.weight": WeightSpec((h, q))}

    def bind(self, tensors, rt) -> None:
        parts = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        # one product for q, k and v: their rows one after the other
        self.w_qkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        qkv = linear(h, self.w_qkv, out_dtype=self.act_dtype)
        fused = self.position.fused() if self.position is not None else (0, 1.0)
        if fused is None:
            self.position.apply(qkv, ctx, self.num_heads, self.num_kv_heads, self.head_dim)
            fused = (0, 1.0)
        rotary_dim, theta = fused
        ops.rope_kv_write(qkv, ctx.positions, ctx.slot_maps[cache.group] if writes else None,
                          cache.k if writes else None, cache.v if writes else None,
                          self.num_heads, self.num_kv_heads, self.head_dim, rotary_dim, theta,
                          write_kv=writes)
        o = ops.attention(qkv, cache.k, cache.v, ctx.block_tables[cache.group], ctx,
                          self.num_heads, self.num_kv_heads, self.head_dim, self.window, self.scale)
        linear(o, self.w_o, accumulate_into=residual)


register_part("mixer", "attention", CausalAttention)
