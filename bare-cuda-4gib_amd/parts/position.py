"""Position encodings applied to queries and keys before keys are cached."""
from __future__ import annotations

from ..errors import ConfigError
from .base import Part, register_part


class Rotary(Part):
    """Rotary positions with the rotate-half pairing (element i with element
    i + dim/2): inv_freq_i = theta^(-2i/dim), angle = position * inv_freq_i,
    (lo, hi) -> (lo cos - hi sin, hi cos + lo sin), angles in float
    (reference: engine/kernels/rope.cu:44-53).  ``dim`` may be smaller than the
    head size; the remaining elements pass through."""
    category = "position"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, theta: float, dim: int):
        if dim <= 0 or dim % 2:
            raise ConfigError(f"rotary: dim must be positive and even, got {dim}")
        if theta <= 0:
            raise ConfigError(f"rotary: theta must be positive, got {theta}")
        self.theta, self.dim = float(theta), int(dim)

    def fused(self):
        return self.dim, self.theta


class NoPosition(Part):
    """No position encoding: queries and keys are used as projected."""
    category = "position"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def fused(self):
        return 0, 1.0


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
