"""One registry from an architecture's name to its model.

The reference hard-codes Llama in ``Model`` (engine/src/model.cpp:314-440) and
has no registry; here config.json's ``architectures[0]`` (with ``model_type``
as a fallback) selects an :class:`Architecture`, which supplies the typed
configuration and the function that turns a configuration into a model
description (layers, schedule, weight names).  Loader, cache manager, step
function, scheduler and the programs never name an architecture.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, List, Tuple, Type

from ..errors import ConfigError
from .base import ModelConfig, read_config_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str                      # config.json "architectures"[0]
    model_type: str                # config.json "model_type"
    config_class: Type[ModelConfig]
    describe: Callable[[ModelConfig], Any]   # config -> engine.ModelSpec
    # glob patterns of tensor names that this architecture's checkpoints may carry and the engine
    # does not need (buffers that are recomputed): passed over without a warning
    ignored_tensors: Tuple[str, ...] = ()


_BY_NAME: Dict[str, Architecture] = {}
_BY_TYPE: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    if not replace and (arch.name in _BY_NAME or arch.model_type in _BY_TYPE):
        raise ConfigError(f"architecture '{arch.name}' / model_type '{arch.model_type}' "
                          "is already registered")
    _BY_NAME[arch.name] = arch
    _BY_TYPE[arch.model_type] = arch
    return arch


def unregister_architecture(name: str) -> None:
    arch = _BY_NAME.pop(name, None)
    if arch is not None:
        _BY_TYPE.pop(arch.model_type, None)


def registered_architectures() -> List[str]:
    return sorted(_BY_NAME)


def architecture_for(raw: Dict[str, Any]) -> Architecture:
    """The registered architecture a parsed config.json names."""
    names = raw.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for n in names:
        if n in _BY_NAME:
            return _BY_NAME[n]
    mt = raw.get("model_type")
    if mt in _BY_TYPE:
        return _BY_TYPE[mt]
    asked = ", ".join(repr(n) for n in names) or "none"
    raise ConfigError(
        f"no registered architecture for architectures=[{asked}], model_type={mt!r}; "
        f"registered: {', '.join(registered_architectures()) or 'none'}")


def load_config(path: str):
    """(architecture, typed configuration) of a model folder or config.json."""
    raw = read_config_json(path)
    arch = architecture_for(raw)
    return arch, arch.config_class.from_dict(raw)
