"""An activation that is the norm of the residual stream, not yet computed.

A block hands ``Normed(x, norm)`` to a mixer or feed-forward that declares
``accepts_lazy_norm``; :func:`parts.linear.linear` then fuses the norm into the
product where a kernel can -- or takes what the product before has prepared for
this norm (``pre``) -- and otherwise calls :meth:`tensor`, which runs the norm
once and keeps the result.
"""
from __future__ import annotations

from typing import Optional

import torch


class Normed:
    def __init__(self, x: torch.Tensor, norm, ctx=None, rows: Optional[torch.Tensor] = None,
                 n_rows: Optional[int] = None, pre=None, done: Optional[torch.Tensor] = None):
        self.x, self.norm, self.ctx, self.rows = x, norm, ctx, rows
        # what the product that last added into x left for this norm (ops.Prenormed), if anything
        self.pre = pre if rows is None else None
        self.n_rows = x.shape[0] if rows is None and n_rows is None else (n_rows if n_rows is not None else rows.numel())
        self._tensor: Optional[torch.Tensor] = done      # (``done``: the product before has computed the norm already)

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, self.ctx, rows=self.rows, n_rows=self.n_rows if self.rows is not None else None)
        return self._tensor

    def fusable_scale(self):
        """(scale vector, eps) if the norm is a plain RMSNorm that a product may absorb, else None."""
        f = getattr(self.norm, "fusable", None)
        return f() if f is not None else None
