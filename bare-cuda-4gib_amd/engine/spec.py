"""A model as data: which parts make each layer, and in which order layers run.

An architecture's ``describe(config)`` returns a :class:`ModelSpec`; nothing
below it knows which architecture it came from.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional


@dataclasses.dataclass
class PartSpec:
    """One part: its registered kind, its sizes and constants, and the prefix
    its tensors carry in the weight file (``rename`` maps a part's own tensor
    names to other file names where an architecture calls them differently)."""
    kind: str
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)
    prefix: str = ""
    rename: Dict[str, str] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class LayerSpec:
    """One layer: an arrangement (``block``) of a mixer, a feed-forward and
    their norms.  Every layer has its own, so layers of one model may differ."""
    block: str
    mixer: PartSpec
    ffn: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec


@dataclasses.dataclass
class ScheduleEntry:
    """One execution of a layer.  ``cache`` names the cache stream its mixer
    uses (any hashable id; entries that share an id share the cache), and
    ``writes`` says whether this execution appends to that stream or only
    reads what another entry wrote."""
    layer: int
    cache: Optional[Any] = None
    writes: bool = True


@dataclasses.dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    max_seq_len: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    head: PartSpec
