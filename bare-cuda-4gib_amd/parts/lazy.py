"""An activation that is the norm of the residual stream, not yet computed.

A block hands ``Normed(x, norm)`` to a mixer or feed-forward that declares
``accepts_lazy_norm``; :func:`parts.linear.linear` then fuses the norm into the
product where a kernel can -- or takes what the product before has prepared for
this norm (``pre``) -- and otherwise calls :meth:`tensor`, which runs the norm
once and keeps the result.
"""
from __future__ import annotations

import contextlib
from typing import Any, Dict, Optional, Tuple

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


class NormHandoff:
    """The whole protocol by which a product that adds into the residual stream prepares the norm that reads the
    stream next, in one place (a step's StepContext carries one).  Three parties use it:

    the model    ``begin_entry(layer, following, n_rows)`` before every schedule entry: what the entry before left
                 for this entry's first norm stays, everything else goes, and the first reader of the entry after
                 this one is noted (``first_reader(n_rows) -> (norm, takes_parts)`` of a block that has one);
                 ``end_step()`` after the last.
    a block      ``with handoff.reader(norm, takes_parts):`` around each part that adds into the stream, naming the
                 norm that reads the stream after that part (``handoff.next_entry`` for its last part), and
                 ``take(norm)`` for what was left for a norm of its own.
    a product    (parts.linear.linear) ``reading_next`` -- (norm, takes_parts) or None -- and ``leave(norm, what)``.

    What is left is the finished norm (ops.Finished), which serves every reader, or -- only for a reader that says
    it takes them -- the parts of one that a product can finish (ops.Prenormed).  Nothing left outlives the entry
    after the one that made it.  A block that does not use any of this stays correct: its norms simply run."""

    def __init__(self):
        self.reading_next: Optional[Tuple[Any, bool]] = None
        self.next_entry: Optional[Tuple[Any, bool]] = None
        self._left: Dict[int, Any] = {}

    @staticmethod
    def _first_reader(layer, n_rows: int) -> Optional[Tuple[Any, bool]]:
        first = getattr(layer, "first_reader", None)
        return first(n_rows) if first is not None else None

    def begin_entry(self, layer, following, n_rows: int) -> None:
        mine = self._first_reader(layer, n_rows)
        kept = self._left.pop(id(mine[0]), None) if mine is not None else None
        self._left.clear()
        if kept is not None:
            self._left[id(mine[0])] = kept
        self.next_entry = self._first_reader(following, n_rows) if following is not None else None
        self.reading_next = None

    def end_step(self) -> None:
        self._left.clear()
        self.next_entry = self.reading_next = None

    @contextlib.contextmanager
    def reader(self, norm, takes_parts: bool = False):
        before = self.reading_next
        self.reading_next = (norm, bool(takes_parts)) if norm is not None else None
        try:
            yield
        finally:
            self.reading_next = before

    def leave(self, norm, what) -> None:
        self._left[id(norm)] = what

    def take(self, norm):
        return self._left.pop(id(norm), None)
