"""Choosing tokens for a step's logits rows on the device."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..csrc import ops
from .params import SamplingParams


class Picked:
    """Tokens chosen on the device and on their way to the host: ``tokens_for(rows)`` is the device
    tensor a following step can take its tokens from, ``result()`` waits for the copy and returns
    the ids."""
    def __init__(self, ids: torch.Tensor):
        self.ids = ids
        self.host = torch.empty(ids.numel(), dtype=torch.int32).pin_memory()
        self.host.copy_(ids, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()

    def tokens_for(self, rows: Sequence[int]) -> torch.Tensor:
        if len(rows) == self.ids.numel():
            return self.ids
        return self.ids[torch.tensor(rows, dtype=torch.int64).to(self.ids.device, non_blocking=True)]

    def result(self) -> List[int]:
        self.copied.synchronize()
        return self.host.tolist()


class DevicePicker:
    """Every row's token is chosen on the device: greedy rows get the argmax (lowest index on ties); rows with a
    temperature are drawn from the request's own uniform number -- by inverse CDF in the order of the ids where
    nothing filters them, and, with top-k or top-p, by the reference's law for those (the tokens by falling weight,
    the k likeliest, the fewest of them that reach top_p, the first at which u of the kept mass is passed:
    engine/src/sampler.cpp:63-104) in a kernel of its own over just those rows.  One small download per step,
    and none before the next step may start (pick_later)."""

    @staticmethod
    def _filters(p: SamplingParams, vocab: int) -> bool:
        """Whether the law for filtered rows applies: a top-k below the vocabulary or a top-p below 1 (with
        neither, the walk is in the order of the ids: sampling/host.py::sample_token)."""
        return 0 < p.top_k < vocab or p.top_p < 1.0

    def _on_device(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> torch.Tensor:
        n, vocab = logits.shape
        assert n == len(params) == len(rngs)
        temps = [0.0] * n
        us = [0.0] * n
        filtered = []
        for i, p in enumerate(params):
            if p.greedy():
                continue
            us[i] = rngs[i].uniform()
            if self._filters(p, vocab):
                filtered.append(i)             # (temperature 0 for the first kernel: it leaves the argmax there)
            else:
                temps[i] = float(p.temperature)
        if any(t > 0.0 for t in temps):
            t_dev = torch.tensor(temps, dtype=torch.float32).to(logits.device, non_blocking=True)
            u_dev = torch.tensor(us, dtype=torch.float64).to(logits.device, non_blocking=True)
            ids = ops.sample(logits, t_dev, u_dev)
        else:
            ids = ops.argmax(logits)
        if filtered:
            dev = logits.device
            # one upload for the rows' numbers: (row, top_k) as int32, (temperature) as float32, (u, top_p) as float64
            ints = torch.tensor([filtered, [params[i].top_k for i in filtered]], dtype=torch.int32).to(dev, non_blocking=True)
            temp = torch.tensor([params[i].temperature for i in filtered], dtype=torch.float32).to(dev, non_blocking=True)
            reals = torch.tensor([[us[i] for i in filtered], [params[i].top_p for i in filtered]],
                                 dtype=torch.float64).to(dev, non_blocking=True)
            ops.sample_filtered(logits, ids, ints[0], temp, reals[0], ints[1], reals[1])
        return ids

    def pick(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> List[int]:
        return [int(t) for t in self._on_device(logits, params, rngs).tolist()]

    def pick_later(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> Optional[Picked]:
        """The same choice without waiting for it: the tokens on the device and on their way to the host."""
        return Picked(self._on_device(logits, params, rngs))
