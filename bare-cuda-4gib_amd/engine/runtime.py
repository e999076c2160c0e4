"""What every part needs to know about where and how it runs."""
from __future__ import annotations

import dataclasses

import torch

from ..errors import EngineError

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise EngineError(f"dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise EngineError(f"dtype must be one of {sorted(_DTYPES)}, got {name!r}") from None


@dataclasses.dataclass
class Runtime:
    """device: where tensors live.  act_dtype: the storage type of activations
    between kernels and of the cache -- bfloat16 (what serving uses; float
    accumulation everywhere, float residual stream and logits) or float32 (a
    true 32-bit path: every weight widened to float, plain float arithmetic, no
    matrix-core mode of reduced precision)."""
    device: torch.device
    act_dtype: torch.dtype

    @property
    def full_precision(self) -> bool:
        return self.act_dtype == torch.float32

    def place_weight(self, t: torch.Tensor) -> torch.Tensor:
        """A loaded tensor on the device: kept as stored (bfloat16 stays
        bfloat16, 32-bit stays 32-bit, integers int32), except that the 32-bit
        path widens everything to float and that a tensor stored in float16 is
        kept in bfloat16 otherwise (rounded to nearest, ties to even: a
        float16 checkpoint then runs on the same kernels as a bfloat16 one)."""
        t = t.to(self.device)
        if t.is_floating_point() and self.full_precision and t.dtype != torch.float32:
            t = t.to(torch.float32)
        elif t.dtype == torch.float16:
            t = t.to(torch.float32).to(torch.bfloat16)
        return t.contiguous()
