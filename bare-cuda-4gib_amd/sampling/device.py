"""Choosing tokens for a step's logits rows on the device."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..csrc import ops
from .host import sample_token
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
    """Greedy rows get the device argmax (lowest index on ties); rows with a
    temperature and no filter are drawn on the device by inverse CDF from the
    request's own uniform number; rows with top-k or top-p are brought to the
    host and drawn there (reference: Scheduler::choose,
    engine/src/scheduler.cpp:96-100).  One small download per step."""

    def _on_device(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence):
        """(ids chosen on the device for every row, rows that the host has to draw instead)."""
        n = logits.shape[0]
        assert n == len(params) == len(rngs)
        temps = [0.0] * n
        us = [0.0] * n
        host_rows = []
        for i, p in enumerate(params):
            if p.greedy():
                continue
            if p.filtered():
                host_rows.append(i)
            else:
                temps[i] = float(p.temperature)
                us[i] = rngs[i].uniform()
        if any(t > 0.0 for t in temps):
            t_dev = torch.tensor(temps, dtype=torch.float32).to(logits.device, non_blocking=True)
            u_dev = torch.tensor(us, dtype=torch.float64).to(logits.device, non_blocking=True)
            return ops.sample(logits, t_dev, u_dev), host_rows
        return ops.argmax(logits), host_rows

    def pick(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> List[int]:
        ids, host_rows = self._on_device(logits, params, rngs)
        tokens = ids.tolist()
        for i in host_rows:
            tokens[i] = sample_token(logits[i].cpu().numpy(), params[i], rngs[i])
        return [int(t) for t in tokens]

    def pick_later(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> Optional[Picked]:
        """The same choice without waiting for it: None if some row has to be drawn on the host
        (top-k, top-p), else the tokens on the device and on their way to the host."""
        if any(p.filtered() and not p.greedy() for p in params):
            return None
        ids, _ = self._on_device(logits, params, rngs)
        return Picked(ids)
