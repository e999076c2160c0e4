"""Sampling options, with the reference's names and meanings
(engine/include/llm/sampler.h:9-25, engine/src/sampler.cpp:20-33)."""
from __future__ import annotations

import dataclasses
import math
import os


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 0.0   # 0 is greedy
    top_p: float = 1.0         # keep the fewest likeliest tokens whose probability reaches top_p
    top_k: int = 0             # keep the k likeliest tokens; 0 keeps all
    seed: int = -1             # -1 draws a random seed

    def greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_k == 1

    def filtered(self) -> bool:
        return self.top_k > 0 or self.top_p < 1.0


def check_sampling(p: SamplingParams) -> str:
    """Empty if the params are valid, else why not."""
    if not isinstance(p.temperature, (int, float)) or not (p.temperature >= 0.0) or not math.isfinite(p.temperature):
        return "temperature must be a finite number >= 0"
    if not (0.0 < p.top_p <= 1.0):
        return "top_p must be in (0, 1]"
    if p.top_k < 0:
        return "top_k must be >= 0"
    return ""


def seed_for(p: SamplingParams) -> int:
    """The seed itself if it is >= 0, else 64 random bits."""
    if p.seed >= 0:
        return int(p.seed)
    return int.from_bytes(os.urandom(8), "little")
