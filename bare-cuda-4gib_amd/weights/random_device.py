"""Random weights made on the device, for measurements: the same law as the
random-weights mode that writes a folder (every matrix and table N(0, std),
norm scales 1.0, rounded to bfloat16 if asked), drawn from the device's
generator seeded with ``seed`` -- so not the same numbers as the folder mode,
which draws on the host."""
from __future__ import annotations

from typing import Dict

import torch

from .loader import WeightSpec


def random_tensors_on_device(expected: Dict[str, WeightSpec], seed: int, dtype: torch.dtype, device,
                             std: float = 0.02) -> Dict[str, torch.Tensor]:
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out = {}
    for name, spec in expected.items():
        if spec.optional:
            continue
        if spec.init == "ones":
            out[name] = torch.ones(spec.shape, dtype=dtype, device=device)
        elif spec.kind == "int_table":
            out[name] = torch.zeros(spec.shape, dtype=torch.int32, device=device)
        else:
            t = torch.empty(spec.shape, dtype=torch.float32, device=device)
            t.normal_(0.0, std, generator=gen)
            out[name] = t.to(dtype)
    return out
