"""Choosing tokens for a step's logits rows on the device."""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..csrc import ops
from .host import sample_token
from .params import SamplingParams


class DevicePicker:
    """Greedy rows get the device argmax (lowest index on ties); rows with a
    temperature and no filter are drawn on the device by inverse CDF from the
    request's own uniform number; rows with top-k or top-p are brought to the
    host and drawn there (reference: Scheduler::choose,
    engine/src/scheduler.cpp:96-100).  One small download per step."""

    def pick(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence) -> List[int]:
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
            t_dev = torch.tensor(temps, dtype=torch.float32).to(logits.device)
            u_dev = torch.tensor(us, dtype=torch.float64).to(logits.device)
            tokens = ops.sample(logits, t_dev, u_dev).tolist()
        else:
            tokens = ops.argmax(logits).tolist()
        for i in host_rows:
            tokens[i] = sample_token(logits[i].cpu().numpy(), params[i], rngs[i])
        return [int(t) for t in tokens]
