"""How a layer's parts are arranged around the residual stream."""
from __future__ import annotations

from .base import Part, register_part


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
        h = self.mixer_norm.forward(x, ctx)
        self.mixer.forward(h, ctx, cache, x, writes)
        h = self.ffn_norm.forward(x, ctx)
        self.ffn.forward(h, ctx, x)


register_part("block", "prenorm", PreNormBlock)
