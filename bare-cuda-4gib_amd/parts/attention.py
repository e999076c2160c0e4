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
from .lazy import Normed
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

    def cache_layout(self):
        """The order in which a head's dimensions lie in the cache (known once weights are bound):
        layers that share a cache stream must agree on it."""
        return getattr(self, "dim_order", None)

    @property
    def step_signature(self):
        """Attention parts of the same head counts, head size and window cut a batch alike: one
        preparation a step serves them all."""
        return ("attention", self.num_heads, self.num_kv_heads, self.head_dim, self.window)

    def prepare_step(self, batch):
        """How the matrix-core kernel will cut this batch's rows into pieces (nothing where the plain
        kernel serves): arrays that go up with the batch, and notes for forward()."""
        if getattr(self, "act_dtype", None) != torch.bfloat16 or self.head_dim % 16 or self.head_dim > 256:
            return {}, None
        return ops.attention_plan(batch, self.num_heads, self.num_kv_heads, self.head_dim, self.window)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        q, kv, h = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim, self.hidden_size
        return {"q_proj.weight": WeightSpec((q, h)), "k_proj.weight": WeightSpec((kv, h)),
                "v_proj.weight": WeightSpec((kv, h)), "o_proj.weight": WeightSpec((h, q))}

    def bind(self, tensors, rt) -> None:
        q, k, v, o = (tensors[n] for n in ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight"))
        dt = torch.float32 if any(p.dtype == torch.float32 for p in (q, k, v)) else q.dtype
        fused = self.position.fused() if self.position is not None else (0, 1.0)
        # For the matrix-core kernels every head's dimensions are reordered in blocks of 16 -- eight
        # dimensions, then their rotation partners -- so that the weight-streaming kernel can rotate and
        # write the cache in its epilogue.  Queries, keys and values all live in that order (scores and
        # outputs do not depend on the order, as long as all agree), and the output projection's
        # columns are reordered to match.
        self.block_pairs = (dt == torch.bfloat16 and o.dtype == torch.bfloat16 and self.head_dim % 16 == 0
                            and fused is not None and fused[0] in (0, self.head_dim))
        self.dim_order = tuple(range(self.head_dim))
        if self.block_pairs:
            d, half = self.head_dim, self.head_dim // 2
            self.dim_order = tuple(8 * b + t if t < 8 else half + 8 * b + (t - 8)
                                   for b in range(d // 16) for t in range(16))
            order = torch.tensor(self.dim_order, device=q.device)
            def rows(w, heads):
                return w.view(heads, d, -1)[:, order, :].reshape(heads * d, -1)
            q, k, v = rows(q, self.num_heads), rows(k, self.num_kv_heads), rows(v, self.num_kv_heads)
            o = o.view(-1, self.num_heads, d)[:, :, order].reshape(-1, self.num_heads * d).contiguous()
        # one product for q, k and v: their rows one after the other
        self.w_qkv = ops.StreamedWeight(torch.cat([p.to(dt) for p in (q, k, v)], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(o)
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        """The products' work, plus attention's own: two products of head_dim per query head and visible
        key, and every visible key and value of every request read once."""
        flops, nbytes = super().step_work(batch, rows, elem)
        pairs = keys = 0
        for s in range(batch.n_seqs):
            cached, new = int(batch.seq_ctx[s]), int(batch.seq_start[s + 1] - batch.seq_start[s])
            if self.window > 0:
                pairs += sum(min(self.window, cached + i + 1) for i in range(new))
                keys += min(cached + new, self.window + new - 1)
            else:
                pairs += new * cached + new * (new + 1) // 2
                keys += cached + new
        return (flops + 4.0 * pairs * self.num_heads * self.head_dim,
                nbytes + 2.0 * keys * self.num_kv_heads * self.head_dim * elem)

    def working_bytes_per_row(self, elem: int) -> float:
        """The products' outputs, the attention output, and the float partial outputs and sums of a row whose
        keys are cut into parts (as many as a prompt's work list may make)."""
        q = self.num_heads * self.head_dim
        return (super().working_bytes_per_row(elem) + q * elem
                + ops.ATTENTION_MAX_PROMPT_SPLITS * (q + 2 * self.num_heads) * 4)

    def wants_prepared_norm(self, n_rows: int) -> bool:
        """Whether the q|k|v product is better served by a norm that the product before prepared than by fusing
        the norm or running it: the weight's own plan says (ops.LinearPlan.wants_prepared)."""
        return self.act_dtype == torch.bfloat16 and self.w_qkv.plan.wants_prepared(n_rows)

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        fused = self.position.fused() if self.position is not None else (0, 1.0)
        rotary_dim, theta = fused if fused is not None else (0, 1.0)
        slot_map = ctx.slot_maps[cache.group] if writes else None
        k_cache, v_cache = (cache.k, cache.v) if writes else (None, None)
        q = None
        if self.block_pairs and fused is not None:
            q = self._fused_qkv(h, ctx, slot_map, k_cache, v_cache, rotary_dim, theta, writes)
        if q is None and self.block_pairs and fused is not None:
            q = self._tiled_qkv(h, ctx, slot_map, k_cache, v_cache, rotary_dim, theta, writes)
        if q is None:
            q = linear(h, self.w_qkv, out_dtype=self.act_dtype)
            if fused is None:
                self.position.apply(q, ctx, self.num_heads, self.num_kv_heads, self.head_dim)
            if self.block_pairs and fused is not None:
                # the angles are the same in every layer: a table made once a step
                table = None
                if rotary_dim > 0:
                    table = ctx.shared(("rope_table", rotary_dim, theta),
                                       lambda: ops.rope_table(ctx.positions, rotary_dim, theta))
                ops.rope_kv_write_blocks(q, table, slot_map, k_cache, v_cache, self.num_heads, self.num_kv_heads,
                                         self.head_dim, write_kv=writes)
            else:
                ops.rope_kv_write(q, ctx.positions, slot_map, k_cache, v_cache, self.num_heads, self.num_kv_heads,
                                  self.head_dim, rotary_dim, theta, write_kv=writes, block_pairs=self.block_pairs)
        arrays, notes = ctx.step_data.get(self.step_signature, ({}, None))
        o = ops.attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx, (arrays, notes) if notes else None,
                          self.num_heads, self.num_kv_heads, self.head_dim, self.window, self.scale)
        linear(o, self.w_o, accumulate_into=residual, ctx=ctx)

    def _tiled_qkv(self, h, ctx, slot_map, k_cache, v_cache, rotary_dim, theta, writes):
        """The q|k|v product of many rows (a prompt portion) with rotation and cache write in the tiled kernel's
        epilogue, the angles from the step's table; None where that kernel does not take the operands."""
        x = h.tensor() if isinstance(h, Normed) else h
        if not ops.gemm_qkv_rope_tiled_supported(x, self.w_qkv, self.head_dim, rotary_dim):
            return None
        table = None
        if rotary_dim > 0:
            table = ctx.shared(("rope_table", rotary_dim, theta), lambda: ops.rope_table(ctx.positions, rotary_dim, theta))
        return ops.gemm_qkv_rope_tiled(x, self.w_qkv, table, slot_map, k_cache, v_cache, self.num_heads, self.num_kv_heads,
                                       self.head_dim, write_kv=writes)

    def _fused_qkv(self, h, ctx, slot_map, k_cache, v_cache, rotary_dim, theta, writes):
        """The q|k|v product with rotation and cache write in its epilogue, where a kernel takes
        the rows (a decode step); None otherwise."""
        args = (ctx.positions, slot_map, k_cache, v_cache, self.num_heads, self.num_kv_heads, self.head_dim,
                rotary_dim, theta, writes)
        if isinstance(h, Normed):
            if (h.pre is not None and h._tensor is None
                    and ops.gemm_qkv_rope_supported(h.pre.xb, h.n_rows, False, self.w_qkv, self.head_dim, rotary_dim)):
                return ops.gemm_qkv_rope(h.pre.xb, None, 0.0, self.w_qkv, *args, pre=h.pre)
            scale = h.fusable_scale() if h._tensor is None and h.rows is None else None
            if scale is not None and ops.gemm_qkv_rope_supported(h.x, h.n_rows, True, self.w_qkv, self.head_dim, rotary_dim):
                return ops.gemm_qkv_rope(h.x, scale[0], scale[1], self.w_qkv, *args)
            if h.n_rows > ops.SKINNY_MAX_ROWS:
                return None       # beyond this kernel's rows: the plain product takes the norm as it comes, prepared or not
            h = h.tensor()
        if ops.gemm_qkv_rope_supported(h, h.shape[0], False, self.w_qkv, self.head_dim, rotary_dim):
            return ops.gemm_qkv_rope(h, None, 0.0, self.w_qkv, *args)
        return None


register_part("mixer", "attention", CausalAttention)
