"""One step's batch, as the parts see it."""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from ..parts.lazy import NormHandoff
from .runtime import Runtime


@dataclasses.dataclass
class HostBatch:
    """A step's batch as the host knows it, before anything is on the device: request s (in batch
    order) brings ``seq_start[s+1] - seq_start[s]`` tokens after ``seq_ctx[s]`` cached ones.  What a
    part's ``prepare_step`` is given.  ``captured``: the step is (or will be replayed from) a captured
    graph -- then ``max_kv_len`` is not this step's longest context but the bound of the graph's context
    bucket, so that whatever launch geometry a part derives from it holds for every replay."""
    n_tokens: int
    n_seqs: int
    seq_start: Sequence[int]             # [S+1]
    seq_ctx: Sequence[int]               # [S] tokens cached before this step
    seq_slots: Sequence[int]             # [S] state slot of each request
    max_q_len: int
    max_kv_len: int
    captured: bool = False


@dataclasses.dataclass
class StepContext:
    """A batch of rows: request s (in batch order) contributes its next
    ``seq_start[s+1] - seq_start[s]`` tokens at positions ``seq_ctx[s] ...``.
    Device tensors are int32.  A mixer reads what it needs: a paged one the
    block table and slot map of its group, one with state of its own the
    requests' slots and where their rows start."""
    rt: Runtime
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor              # [T] device
    positions: torch.Tensor              # [T] device: absolute position of each row
    row_seq: torch.Tensor                # [T] device: which request of the batch a row belongs to
    seq_start: List[int]                 # [S+1] host
    seq_ctx: List[int]                   # [S] host: tokens cached before this step
    seq_slots: List[int]                 # [S] host: state slot of each request
    seq_start_dev: torch.Tensor          # [S+1] device
    seq_ctx_dev: torch.Tensor            # [S] device
    seq_slots_dev: torch.Tensor          # [S] device
    logit_rows: torch.Tensor             # [n_logits] device: rows whose logits are wanted
    n_logits: int
    block_tables: Dict[Hashable, torch.Tensor]   # group -> [S, max_pages] device
    slot_maps: Dict[Hashable, torch.Tensor]      # group -> [T] device: page*page_tokens + offset
    max_q_len: int
    max_kv_len: int
    cache_views: Dict[Hashable, Any] = dataclasses.field(default_factory=dict)
    made: Dict[Any, Any] = dataclasses.field(default_factory=dict)      # see shared()
    # What the parts' prepare_step made of this batch, by the part's step_signature: (int32 device
    # tensors by name -- they came up with the batch's own arrays, in the same copy --, whatever else
    # the part noted for itself on the host).
    step_data: Dict[Hashable, Tuple[Dict[str, torch.Tensor], Any]] = dataclasses.field(default_factory=dict)
    captured: bool = False               # see HostBatch
    # Who reads the residual stream next and what the product before left for that reader: see NormHandoff.
    handoff: NormHandoff = dataclasses.field(default_factory=NormHandoff)

    def cache(self, stream: Optional[Hashable]):
        return None if stream is None else self.cache_views.get(stream)

    def shared(self, key, make):
        """What several layers of one step share (a table of rotation angles, say): made by the
        first that asks, kept until the step ends."""
        if key not in self.made:
            self.made[key] = make()
        return self.made[key]
