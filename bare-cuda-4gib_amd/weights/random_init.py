"""Random-weights mode: a model folder from a configuration and a seed.

Every matrix and table is N(0, std) with std 0.02 and every norm scale is 1.0;
values are drawn in float32 from torch's CPU generator seeded with ``seed``,
tensor after tensor in the order the model's parts declare them, and rounded
to bfloat16 (to nearest, ties to even) when ``dtype`` is bfloat16.  (The
reference only has random weights in its Python fixture generator,
tools/references/reference_forward.py:301-321: matrices randn * 0.05, norm
scales 1 + 0.05 * randn.)  Two options make folders on which more can go
wrong: ``norm_std`` draws every norm scale as 1 + norm_std * randn, a draw of
its own for every norm, and ``scales`` multiplies the tensors whose names match
a pattern by a factor (larger query and key weights make attention peaked).
"""
from __future__ import annotations

import fnmatch
import json
import os
from typing import Any, Dict, Optional, Union

import torch

from ..config.base import ModelConfig
from ..config.registry import architecture_for
from ..errors import ConfigError
from .safetensors_io import SafetensorsWriter

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def random_tensor(spec, gen: torch.Generator, std: float, dtype: torch.dtype, norm_std: float = 0.0,
                  factor: float = 1.0) -> torch.Tensor:
    if spec.init == "ones":
        if norm_std == 0.0:
            return torch.full(spec.shape, factor, dtype=dtype)
        return ((1.0 + norm_std * torch.randn(spec.shape, generator=gen, dtype=torch.float32)) * factor).to(dtype)
    if spec.kind == "int_table":
        return torch.zeros(spec.shape, dtype=torch.int32)
    return (torch.randn(spec.shape, generator=gen, dtype=torch.float32) * (std * factor)).to(dtype)


def write_random_model(config: Union[Dict[str, Any], ModelConfig], seed: int, out_dir: str,
                       dtype: str = "bfloat16", std: float = 0.02, norm_std: float = 0.0,
                       scales: Optional[Dict[str, float]] = None) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors``; returns out_dir.
    ``norm_std``: spread of the norm scales around 1.0 (0: exactly 1.0).  ``scales``: glob pattern
    of tensor names -> factor on what is drawn for them (the first pattern that matches)."""
    from ..engine.model import expected_weights

    if dtype not in _DTYPES:
        raise ConfigError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}")
    tdtype = _DTYPES[dtype]
    raw = config.to_dict() if isinstance(config, ModelConfig) else dict(config)
    arch = architecture_for(raw)
    cfg = arch.config_class.from_dict(raw)
    raw = dict(raw)
    raw.setdefault("architectures", [arch.name])
    raw.setdefault("model_type", arch.model_type)
    raw["torch_dtype"] = "bfloat16" if tdtype == torch.bfloat16 else "float32"
    spec = arch.describe(cfg)
    expected = {n: s for n, s in expected_weights(spec).items() if not s.optional}
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(raw, fh, indent=1)
    layout = [(n, s.shape, torch.int32 if s.kind == "int_table" else tdtype) for n, s in expected.items()]
    writer = SafetensorsWriter(os.path.join(out_dir, "model.safetensors"), layout,
                               metadata={"format": "pt", "seed": seed, "std": std, "norm_std": norm_std})
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    scales = scales or {}

    def factor(name: str) -> float:
        for pattern, f in scales.items():
            if fnmatch.fnmatchcase(name, pattern):
                return float(f)
        return 1.0
    for name, s in expected.items():
        writer.write(name, random_tensor(s, gen, std, tdtype, norm_std, factor(name)))
    writer.close()
    return out_dir
