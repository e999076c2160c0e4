"""How a layer's parts are arranged around the residual stream."""
from __future__ import annotations

from ..csrc import ops
from .base import Part, register_part
from .lazy import Normed


class PreNormBlock(Part):
    """x += mixer(norm(x)); x += ffn(norm(x))  (reference: engine/src/model.cpp:526-604).
    The residual stream x is float32 and is updated in place."""
    category = "block"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, mixer, ffn, mixer_norm, ffn_norm):
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    def children(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def forward(self, x, ctx, cache, writes: bool = True) -> None:
        # Each part is told which norm reads the stream after it, so that its last product can prepare that
        # norm: the feed-forward's after the mixer, the next entry's first after the feed-forward.
        handoff, n = ctx.handoff, x.shape[0]
        with handoff.reader(self.ffn_norm, self._wants_prepared(self.ffn, n)):
            self.mixer.forward(self._normed(self.mixer, self.mixer_norm, x, ctx), ctx, cache, x, writes)
        with handoff.reader(*(handoff.next_entry or (None, False))):
            self.ffn.forward(self._normed(self.ffn, self.ffn_norm, x, ctx), ctx, x)

    def first_reader(self, n_rows: int):
        """(the norm this block begins with, whether its reader takes the parts of a prepared norm for a step of
        ``n_rows`` rows): what the entry before may prepare."""
        return self.mixer_norm, self._wants_prepared(self.mixer, n_rows)

    @staticmethod
    def _wants_prepared(part, n_rows: int) -> bool:
        """Whether the part's first product is better served by a prepared norm than by fusing the
        norm or running it (parts that do not say are not: nothing is prepared for them)."""
        wants = getattr(part, "wants_prepared_norm", None)
        return bool(wants(n_rows)) if wants is not None else False

    @staticmethod
    def _normed(part, norm, x, ctx):
        """The part's input: the norm's result, or -- for a part that says it takes one -- the
        norm not yet computed, so that the part's first product can absorb it (or take what the
        product before has prepared for it)."""
        pre = ctx.handoff.take(norm)
        if isinstance(pre, ops.Finished):
            return Normed(x, norm, ctx, done=pre.tensor) if getattr(part, "accepts_lazy_norm", False) else pre.tensor
        if getattr(part, "accepts_lazy_norm", False):
            return Normed(x, norm, ctx, pre=pre)
        return norm.forward(x, ctx)


register_part("block", "prenorm", PreNormBlock)
