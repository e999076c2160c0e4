"""The step function: one batch of (request, its next tokens) through the
model, from the cache, returning logits at the wanted places.

(Reference: Model::forward_rows, engine/src/model.cpp:442-616 -- rows grouped
by slot, positions = cached length + offset, pages reserved before anything
runs, lengths advanced after the last layer.  The reference computes logits for
every row; here only the wanted rows reach the final norm and the output
projection.)
"""
from __future__ import annotations

import dataclasses
from typing import Hashable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..errors import EngineError
from .batch import StepContext
from .model import Model


@dataclasses.dataclass
class StepEntry:
    """A request's next tokens, and the places among them (0-based) whose
    logits are wanted."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class Executor:
    """Owns a model's cache and runs steps on it.

    page_tokens: tokens per cache page.  num_pages: pages in each group's
    pool.  max_requests: requests that can be live at once.  max_tokens: the
    most tokens one request may hold.  max_batch_tokens: the most rows one
    step may bring (0: no limit but memory).
    """

    def __init__(self, model: Model, *, num_pages: int, max_requests: int, max_tokens: int,
                 page_tokens: int = 64, max_batch_tokens: int = 0, poison: bool = False):
        if model.rt is None:
            raise EngineError("executor: the model has no weights bound")
        self.model = model
        self.rt = model.rt
        self.max_batch_tokens = max_batch_tokens
        self.cache = CacheManager(model.cache_streams(), page_tokens=page_tokens, num_pages=num_pages,
                                  max_requests=max_requests, max_tokens=max_tokens,
                                  dtype=self.rt.act_dtype, device=self.rt.device, poison=poison)
        self._views = {sid: self.cache.view(sid) for sid in self.cache.specs}

    # ---- requests -----------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        return self.cache.admit(request)

    def release(self, request: Hashable) -> None:
        self.cache.release(request)

    def has(self, request: Hashable) -> bool:
        return self.cache.has(request)

    def length(self, request: Hashable) -> int:
        return self.cache.length(request)

    # ---- the step -----------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> int:
        if not entries:
            raise EngineError("step: no entries")
        seen = set()
        total = 0
        vocab = self.model.vocab_size
        for e in entries:
            if not self.cache.has(e.request):
                raise EngineError(f"step: unknown request {e.request!r}")
            if e.request in seen:
                raise EngineError(f"step: request {e.request!r} appears twice")
            seen.add(e.request)
            n = len(e.tokens)
            if n == 0:
                raise EngineError(f"step: request {e.request!r} brings no tokens")
            for t in e.tokens:
                if not (0 <= int(t) < vocab):
                    raise EngineError(f"step: token id {t} of request {e.request!r} is outside [0, {vocab})")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise EngineError(f"step: wanted place {w} of request {e.request!r} is outside its {n} tokens")
            total += n
        if self.max_batch_tokens and total > self.max_batch_tokens:
            raise EngineError(f"step: {total} rows are more than max_batch_tokens={self.max_batch_tokens}")
        return total

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Host arrays of the batch, uploaded in one copy."""
        cache, P = self.cache, self.cache.page_tokens
        token_ids: List[int] = []
        positions: List[int] = []
        row_seq: List[int] = []
        seq_start, seq_ctx, seq_slots, logit_rows = [0], [], [], []
        max_q = max_kv = 0
        for s, e in enumerate(entries):
            n, ctx_len = len(e.tokens), cache.length(e.request)
            base = seq_start[-1]
            token_ids.extend(int(t) for t in e.tokens)
            positions.extend(range(ctx_len, ctx_len + n))
            row_seq.extend([s] * n)
            seq_start.append(base + n)
            seq_ctx.append(ctx_len)
            seq_slots.append(cache.slot(e.request))
            logit_rows.extend(base + int(w) for w in e.want)
            max_q, max_kv = max(max_q, n), max(max_kv, ctx_len + n)
        T, S = len(token_ids), len(entries)
        flat = token_ids + positions + row_seq + seq_start + seq_ctx + seq_slots + logit_rows
        layout = {"token_ids": T, "positions": T, "row_seq": T, "seq_start": S + 1, "seq_ctx": S,
                  "seq_slots": S, "logit_rows": len(logit_rows)}
        group_layout = []
        for g in cache.groups:
            tables = [cache.table(g, e.request) for e in entries]
            width = max(1, max(len(t) for t in tables))
            for t in tables:
                flat.extend(t)
                flat.extend([-1] * (width - len(t)))
            slot_map = []
            for e, t in zip(entries, tables):
                ctx_len = cache.length(e.request)
                for p in range(ctx_len, ctx_len + len(e.tokens)):
                    slot_map.append(t[p // P] * P + p % P)
            flat.extend(slot_map)
            group_layout.append((g, width))
        dev = torch.tensor(flat, dtype=torch.int32).to(self.rt.device, non_blocking=True)
        off = 0
        parts = {}
        for name, n in layout.items():
            parts[name] = dev[off:off + n]
            off += n
        block_tables, slot_maps = {}, {}
        for g, width in group_layout:
            block_tables[g] = dev[off:off + S * width].view(S, width)
            off += S * width
            slot_maps[g] = dev[off:off + T]
            off += T
        return StepContext(
            rt=self.rt, n_tokens=T, n_seqs=S, token_ids=parts["token_ids"], positions=parts["positions"],
            row_seq=parts["row_seq"], seq_start=seq_start, seq_ctx=seq_ctx, seq_slots=seq_slots,
            seq_start_dev=parts["seq_start"], seq_ctx_dev=parts["seq_ctx"], seq_slots_dev=parts["seq_slots"],
            logit_rows=parts["logit_rows"], n_logits=len(logit_rows), block_tables=block_tables,
            slot_maps=slot_maps, max_q_len=max_q, max_kv_len=max_kv, cache_views=self._views)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run the entries as one batch.  Returns float32 logits
        [number of wanted places, vocab] on the device, in the order of the
        entries and of their ``want`` lists; None if nothing is wanted.

        Raises OutOfPages, with nothing changed, if the cache cannot hold the
        batch's tokens."""
        self._validate(entries)
        self.cache.reserve([(e.request, len(e.tokens)) for e in entries])
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx)
        for e in entries:
            self.cache.advance(e.request, len(e.tokens))
        return logits
