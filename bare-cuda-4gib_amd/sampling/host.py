"""Sampling on the host, with the reference's law (engine/src/sampler.cpp:36-104):
unnormalized weights exp((l - max) / T) in float, their total in double, one
uniform u per token; without filters the token is the first one, walking the
vocabulary in order, at which u * total minus the running sum turns negative;
with top-k / top-p the likeliest tokens (lower id first on ties) are walked
instead, top-p being measured on the top-k set."""
from __future__ import annotations

import numpy as np

from .params import SamplingParams


def sample_weights(logits: np.ndarray, temperature: float) -> np.ndarray:
    logits = np.asarray(logits, dtype=np.float32)
    inv_t = np.float32(1.0) / np.float32(temperature)
    return np.exp((logits - logits.max()) * inv_t).astype(np.float32)


def _argmax(logits: np.ndarray) -> int:
    return int(np.argmax(logits))   # first maximum


def sample_token(logits, params: SamplingParams, rng) -> int:
    """Draw one token id from a row of logits; ``rng.uniform()`` gives u in [0, 1)."""
    logits = np.asarray(logits, dtype=np.float32)
    vocab = logits.shape[0]
    if params.greedy():
        return _argmax(logits)
    w = sample_weights(logits, params.temperature)
    w64 = w.astype(np.float64)
    total = float(w64.sum())
    k = min(params.top_k, vocab) if params.top_k > 0 else vocab
    top_p = params.top_p < 1.0
    if k == vocab and not top_p:
        target = rng.uniform() * total
        hit = np.nonzero(target - np.cumsum(w64) < 0.0)[0]
        return int(hit[0]) if hit.size else _argmax(logits)
    order = np.lexsort((np.arange(vocab), -w64))      # likeliest first, lower id on ties
    kept = order[:k]
    keep = k
    if top_p:
        kept_total = float(w64[kept].sum())
        cum = np.cumsum(w64[kept])
        reach = np.nonzero(cum >= params.top_p * kept_total)[0]
        keep = int(reach[0]) + 1 if reach.size else k   # rounding may leave the sum a hair short
    kept = kept[:keep]
    mass = float(w64[kept].sum())
    target = rng.uniform() * mass
    hit = np.nonzero(target - np.cumsum(w64[kept]) < 0.0)[0]
    return int(kept[hit[0]]) if hit.size else int(kept[-1])
