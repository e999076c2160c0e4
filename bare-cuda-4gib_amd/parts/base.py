"""Parts and their registry.

A part is built from its sizes and constants alone (``PartSpec.params``); it
declares the tensors it needs, receives them once they are on the device, and
runs on whatever batch it is handed.  No part knows which model it is in.

Interfaces, by category (``ctx`` is the step's StepContext, ``x`` the float32
residual stream [T, hidden], ``h`` an activation [T, hidden] in the runtime's
activation dtype):

norm         forward(x, ctx, rows=None, n_rows=None) -> h       (rows: int32 row indices)
position     fused() -> (rotary_dim, theta) for the fused rotate-and-store kernel, or
             None, in which case apply(qkv, ctx, n_heads, n_kv_heads, head_dim) rotates
             q and k in place
mixer        cache_spec() -> PagedKV | FixedState | None
             forward(h, ctx, cache_view, residual, writes) -- adds its output to residual
feedforward  forward(h, ctx, residual) -- adds its output to residual
block        built from (mixer, ffn, mixer_norm, ffn_norm); forward(x, ctx, cache_view, writes)
embedding    forward(ctx) -> x
head         forward(h) -> float32 logits [rows, vocab]
"""
from __future__ import annotations

from typing import Callable, Dict, List

import torch

from ..errors import ConfigError
from ..weights.loader import WeightSpec

_REGISTRY: Dict[str, Dict[str, Callable[..., "Part"]]] = {}


class Part:
    """Base of every part.  Subclasses set ``category``; a part whose forward only launches
    kernels on the current stream (no host reads of device data, no host-side decisions that
    depend on the batch's values) may set ``graph_safe`` so that decode steps can be captured."""
    category = ""
    graph_safe = False

    def weight_specs(self) -> Dict[str, WeightSpec]:
        """Own tensor name (e.g. ``q_proj.weight``) -> what is expected of it."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], rt) -> None:
        """Receive the tensors (on the device) and pack them for the kernels."""

    def children(self) -> List["Part"]:
        return []

    def step_work(self, batch, rows: int, elem: int):
        """(floating-point operations, bytes that have to be read at least) of this part in a step
        in which ``rows`` rows pass through it (``batch``: the step's HostBatch; ``elem``: bytes of a
        stored element).  By default what the part's tensors say: a linear map's weight is read once
        and takes two operations per row and element, a vector is read once, of a table one row per
        row; nested parts add theirs.  A part with work beyond its tensors (attention over a cache)
        adds it."""
        flops = nbytes = 0.0
        for spec in self.weight_specs().values():
            n = 1
            for d in spec.shape:
                n *= d
            if spec.kind == "matrix":
                flops += 2.0 * rows * n
                nbytes += n * elem
            elif spec.kind == "vector":
                nbytes += n * elem
            else:
                nbytes += rows * (n // max(spec.shape[0], 1)) * elem
        for child in self.children():
            f, b = child.step_work(batch, rows, elem)
            flops, nbytes = flops + f, nbytes + b
        return flops, nbytes

    def working_bytes_per_row(self, elem: int) -> float:
        """Device bytes this part needs for every row of a step while it runs, beyond its weights and the
        cache (``elem``: bytes of a stored activation): by default the output of every linear map it holds,
        nested parts included -- an upper bound, since what one product leaves is mostly gone before the
        part's last product runs.  A part with working memory that its tensors do not show (float partial
        results, staging) adds it."""
        total = 0.0
        for spec in self.weight_specs().values():
            if spec.kind == "matrix" and len(spec.shape) == 2:
                total += spec.shape[0] * elem
        return total + sum(child.working_bytes_per_row(elem) for child in self.children())


def register_part(category: str, kind: str, factory: Callable[..., Part], *, replace: bool = False) -> None:
    """Make ``kind`` buildable: ``factory(**params)`` returns the part."""
    table = _REGISTRY.setdefault(category, {})
    if kind in table and not replace:
        raise ConfigError(f"{category} part '{kind}' is already registered")
    table[kind] = factory


def registered_parts(category: str) -> List[str]:
    return sorted(_REGISTRY.get(category, {}))


def build_part(category: str, spec) -> Part:
    table = _REGISTRY.get(category, {})
    if spec.kind not in table:
        raise ConfigError(f"no {category} part named '{spec.kind}'; registered: "
                          f"{', '.join(sorted(table)) or 'none'}")
    return table[spec.kind](**spec.params)
