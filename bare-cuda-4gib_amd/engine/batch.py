"""One step's batch, as the parts see it."""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Hashable, List, Optional

import torch

from .runtime import Runtime


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

    def cache(self, stream: Optional[Hashable]):
        return None if stream is None else self.cache_views.get(stream)
