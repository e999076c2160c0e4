"""How a layer's parts are arranged around the residual stream."""
from __future__ import annotations

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
        self.mixer.forward(self._normed(self.mixer, self.mixer_norm, x, ctx), ctx, cache, x, writes)
        self.ffn.forward(self._normed(self.ffn, self.ffn_norm, x, ctx), ctx, x)

    @staticmethod
    def _normed(part, norm, x, ctx):
        """The part's input: the norm's result, or -- for a part that says it takes one -- the
        norm not yet computed, so that the part's first product can absorb it."""
        if getattr(part, "accepts_lazy_norm", False):
            return Normed(x, norm, ctx)
        return norm.forward(x, ctx)


register_part("block", "prenorm", PreNormBlock)
