"""Loading weights by tensor name against what the model's parts declare.

The reference validates every tensor by name, dtype and element count and
names the tensor in the message (engine/src/model.cpp:24-74), and it only
looks up the names it needs: a tensor nobody asks for is ignored
(engine/src/loader.cpp:137-148).  Here all problems of a model folder are
collected and reported in one error that lists missing tensors, wrong shapes
and, beside them, the unexpected tensors (a misspelt name shows up as one
missing and one unexpected).  A folder whose only oddity is unexpected tensors
loads, with one warning on standard error that lists them.
"""
from __future__ import annotations

import dataclasses
import fnmatch
import sys
from typing import Dict, Iterable, Tuple

import torch

from ..errors import WeightError
from .safetensors_io import open_model_tensors


@dataclasses.dataclass(frozen=True)
class WeightSpec:
    """What a part expects of one tensor.

    kind: ``matrix`` (a linear map's [out, in] weight), ``vector`` (a norm's
    scale and the like), ``table`` (rows looked up by index) or ``int_table``
    (integer table, kept as int32).  ``init`` is what the random-weights mode
    writes: ``normal`` (N(0, std)) or ``ones``.  An ``optional`` tensor may be
    absent (a tied output head).
    """
    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    optional: bool = False


def _kept_dtype_ok(spec: WeightSpec, t: torch.Tensor) -> bool:
    if spec.kind == "int_table":
        return t.dtype == torch.int32
    return t.dtype in (torch.bfloat16, torch.float32, torch.float16)


def load_weights(model_dir: str, expected: Dict[str, WeightSpec],
                 ignore: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    """Read every expected tensor from ``model_dir``.

    Returns name -> CPU tensor (bfloat16 stays bfloat16, 32-bit stays 32-bit, float16 stays
    float16 until it is placed on the device, where the 16-bit path keeps it in bfloat16,
    integers are int32).  ``ignore`` holds glob patterns of tensor names a file
    may carry that the engine does not need (an architecture names them); they are
    passed over in silence.  Raises one WeightError that lists every missing tensor
    and wrong shape, and the unexpected tensors beside them; unexpected tensors alone
    are a warning.
    """
    available = open_model_tensors(model_dir)
    ignore = tuple(ignore)
    missing, wrong, unexpected = [], [], []
    for name, spec in expected.items():
        if name not in available:
            if not spec.optional:
                missing.append(name)
            continue
        f, n = available[name]
        if tuple(f.shape(n)) != tuple(spec.shape):
            wrong.append(f"{name}: file has {list(f.shape(n))}, the configuration needs {list(spec.shape)}")
        elif spec.kind == "int_table" and not f.stored_dtype(n).startswith(("I", "U")):
            wrong.append(f"{name}: file has dtype {f.stored_dtype(n)}, an integer table is needed")
        elif spec.kind != "int_table" and f.stored_dtype(n) not in ("F32", "F16", "BF16", "F64"):
            wrong.append(f"{name}: file has dtype {f.stored_dtype(n)}, a floating-point tensor is needed")
    for name in available:
        if name not in expected and not any(fnmatch.fnmatchcase(name, pat) for pat in ignore):
            unexpected.append(name)
    if unexpected and not (missing or wrong):
        print(f"[weights] warning: {model_dir} holds {len(unexpected)} tensors the configuration does not "
              f"ask for (ignored): " + ", ".join(sorted(unexpected)), file=sys.stderr, flush=True)
    if missing or wrong:
        lines = [f"weights in {model_dir} do not fit the configuration:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(sorted(missing)))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(sorted(unexpected)))
        if wrong:
            lines.append(f"  wrong shape or dtype ({len(wrong)}):")
            lines.extend("    " + w for w in wrong)
        raise WeightError("\n".join(lines))
    out: Dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        if name in available:
            f, n = available[name]
            t = f.tensor(n)
            assert _kept_dtype_ok(spec, t), (name, t.dtype)
            out[name] = t
    for f in {id(f): f for f, _ in available.values()}.values():
        f.close()
    return out
