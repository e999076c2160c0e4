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
    # tokens per attention tile -> (device int32 [S+1] first tile of each request, number of tiles)
    tiles: Dict[int, Any] = dataclasses.field(default_factory=dict)
    made: Dict[Any, Any] = dataclasses.field(default_factory=dict)      # see shared()
    fixed_attention_splits: int = 0      # non-zero: the key split count is fixed (a captured step)
    # The norm that reads the residual stream next, while a part that adds into the stream runs (set by
    # the block around the part; by the model: the norm the next schedule entry begins with).  A product
    # that adds into the stream may then prepare that norm and leave the result in ``prepared`` under
    # id(norm part); the block hands it to the norm's consumer.  Nothing prepared outlives the entry
    # after the one that made it.
    norm_after: Any = None
    next_entry_norm: Any = None
    prepared: Dict[int, Any] = dataclasses.field(default_factory=dict)

    def cache(self, stream: Optional[Hashable]):
        return None if stream is None else self.cache_views.get(stream)

    def shared(self, key, make):
        """What several layers of one step share (a table of rotation angles, say): made by the
        first that asks, kept until the step ends."""
        if key not in self.made:
            self.made[key] = make()
        return self.made[key]

    def attention_tiles(self, tokens_per_tile: int, short: Optional[bool] = None, short_max: int = 0):
        """Each request's rows cut into tiles of ``tokens_per_tile`` tokens: (first tile of each
        request as a device tensor, total).  With ``short`` given, only the requests that bring at
        most ``short_max`` rows (True) or more than that (False) get tiles; the others get none.
        Made once per step, tile size and choice."""
        key = tokens_per_tile if short is None else (tokens_per_tile, short, short_max)
        if key not in self.tiles:
            starts = [0]
            for s in range(self.n_seqs):
                n = self.seq_start[s + 1] - self.seq_start[s]
                if short is not None and (n <= short_max) != short:
                    n = 0
                starts.append(starts[-1] + -(-n // tokens_per_tile))
            dev = torch.tensor(starts, dtype=torch.int32).to(self.token_ids.device, non_blocking=True)
            self.tiles[key] = (dev, starts[-1])
        return self.tiles[key]
