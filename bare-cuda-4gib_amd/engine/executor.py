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

import numpy as np
import torch

import collections

from ..cache.manager import CacheManager
from ..errors import EngineError
from .batch import HostBatch, StepContext
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
    step may bring (0: no limit but memory).  max_tokens beyond the positions the model's configuration
    gives is refused.

    What a part may add to a step (both optional; the executor knows no part by name):
      prepare_step(batch: HostBatch) -> (arrays, notes)   called once a step before anything is launched,
          also before every replay of a captured step.  ``arrays``: name -> ints, which go up to the
          device in the batch's one copy; ``notes``: anything the part wants to find again.  forward()
          finds both in ``ctx.step_data[part.step_signature]`` (parts with equal ``step_signature``
          share one call; a part without the attribute is its own).  In a captured step only the
          arrays' values may change from replay to replay, not their lengths, and forward() is not run.
      prepare_capture(n_seqs, max_context)                  called once before a decode step of n_seqs
          requests is captured for contexts up to max_context: launch geometry of the part's own is
          fixed here (what forward() derives from ctx.max_kv_len is fixed by itself: that is
          max_context while capturing).
    """
    MAX_GRAPHS = 32       # captured decode graphs kept (each owns its logits and activations); the least
                          # recently used one goes when another is captured
    # A captured decode step has one of these numbers of rows: a step of S requests runs in the smallest graph
    # that holds them, and the rows beyond S stand for no request (they write the cache's scratch page and the
    # scratch slot, and their logits are dropped).  So the graphs a workload needs are bounded by sizes x context
    # buckets however its number of live requests wanders.  Up to 8 rows every count has its own graph: there a
    # row more or less is a kernel form more or less (the norm fused into the products), and a request decoding
    # alone should not pay for rows it does not have.
    GRAPH_ROWS = (1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024)

    def __init__(self, model: Model, *, num_pages: int, max_requests: int, max_tokens: int,
                 page_tokens: int = 64, max_batch_tokens: int = 0, poison: bool = False,
                 use_graphs: bool = True, graph_max_batch: int = 256, beyond_positions: bool = False):
        if model.rt is None:
            raise EngineError("executor: the model has no weights bound")
        # (reference: Model::load, engine/src/model.cpp:429-433.  ``beyond_positions``: a program that replays given
        # ids and serves nobody may say that it wants positions the configuration does not promise -- nothing here
        # keeps a table of them -- and takes the answers for what they are.)
        if max_tokens > model.max_seq_len and not beyond_positions:
            raise EngineError(f"executor: max_tokens {max_tokens} is beyond the model's {model.max_seq_len} positions")
        self.model = model
        self.rt = model.rt
        self.max_batch_tokens = max_batch_tokens
        self.cache = CacheManager(model.cache_streams(), page_tokens=page_tokens, num_pages=num_pages,
                                  max_requests=max_requests, max_tokens=max_tokens,
                                  dtype=self.rt.act_dtype, device=self.rt.device, poison=poison)
        self._views = {sid: self.cache.view(sid) for sid in self.cache.specs}
        parts = model.all_parts()
        # parts that prepare something of their own for every step, one per signature
        self._preparers = {}
        for p in parts:
            if hasattr(p, "prepare_step"):
                self._preparers.setdefault(getattr(p, "step_signature", id(p)), p)
        self._capture_parts = [p for p in parts if hasattr(p, "prepare_capture")]
        # decode steps are replayed from captured graphs if every part of the model allows it
        self.use_graphs = bool(use_graphs) and all(getattr(p, "graph_safe", False) for p in parts) \
            and self.rt.device.type == "cuda"
        self.graph_max_batch = graph_max_batch
        self._graphs = collections.OrderedDict()
        self.captures = 0                 # graphs captured so far (a key captured again after it was dropped counts again)

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
            if n <= 8:
                bad = [t for t in e.tokens if not (0 <= int(t) < vocab)]
            else:                                       # (a prompt portion: looked at as one array)
                ids = np.asarray(e.tokens, dtype=np.int64)
                bad = ids[(ids < 0) | (ids >= vocab)]
            if len(bad):
                raise EngineError(f"step: token id {bad[0]} of request {e.request!r} is outside [0, {vocab})")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise EngineError(f"step: wanted place {w} of request {e.request!r} is outside its {n} tokens")
            total += n
        if self.max_batch_tokens and total > self.max_batch_tokens:
            raise EngineError(f"step: {total} rows are more than max_batch_tokens={self.max_batch_tokens}")
        return total

    def _host_arrays(self, entries: Sequence[StepEntry], table_width: int = 0, all_logits: bool = False,
                     max_kv_bound: int = 0, pad_to: int = 0):
        """The batch as one flat int32 array and the layout of its parts.  ``table_width`` 0
        makes block tables as wide as the batch needs; ``all_logits`` asks for every row;
        ``max_kv_bound`` (a step about to be captured): the context bound the parts are to plan for;
        ``pad_to``: the number of requests the batch is filled up to with rows that stand for no request
        (one token each, nothing cached, the cache's scratch slot and scratch page)."""
        cache, P = self.cache, self.cache.page_tokens
        i32 = np.int32
        token_ids, positions, row_seq, logit_rows = [], [], [], []
        seq_start, seq_ctx, seq_slots = [0], [], []
        max_q = max_kv = 0
        for s, e in enumerate(entries):                 # (whole arrays per request: no Python loop over tokens)
            n, ctx_len = len(e.tokens), cache.length(e.request)
            base = seq_start[-1]
            token_ids.append(np.asarray(e.tokens, dtype=np.int64).astype(i32))
            positions.append(np.arange(ctx_len, ctx_len + n, dtype=i32))
            row_seq.append(np.full(n, s, dtype=i32))
            seq_start.append(base + n)
            seq_ctx.append(ctx_len)
            seq_slots.append(cache.slot(e.request))
            logit_rows.append(np.arange(base, base + n, dtype=i32) if all_logits
                              else base + np.asarray(e.want, dtype=np.int64).astype(i32))
            max_q, max_kv = max(max_q, n), max(max_kv, ctx_len + n)
        n_real = len(entries)
        for s in range(n_real, pad_to):
            base = seq_start[-1]
            token_ids.append(np.zeros(1, dtype=i32))
            positions.append(np.zeros(1, dtype=i32))
            row_seq.append(np.full(1, s, dtype=i32))
            seq_start.append(base + 1)
            seq_ctx.append(0)
            seq_slots.append(cache.scratch_slot)
            logit_rows.append(np.arange(base, base + 1, dtype=i32) if all_logits else np.zeros(0, dtype=i32))
        T, S = seq_start[-1], max(n_real, pad_to)
        empty = np.zeros(0, dtype=i32)
        logit_rows = np.concatenate(logit_rows) if logit_rows else empty
        chunks = [np.concatenate(token_ids) if token_ids else empty, np.concatenate(positions) if positions else empty,
                  np.concatenate(row_seq) if row_seq else empty, np.asarray(seq_start, dtype=i32),
                  np.asarray(seq_ctx, dtype=i32), np.asarray(seq_slots, dtype=i32), logit_rows]
        layout = [("token_ids", T), ("positions", T), ("row_seq", T), ("seq_start", S + 1), ("seq_ctx", S),
                  ("seq_slots", S), ("logit_rows", len(logit_rows))]
        batch = HostBatch(n_tokens=T, n_seqs=S, seq_start=seq_start, seq_ctx=seq_ctx, seq_slots=seq_slots,
                          max_q_len=max_q, max_kv_len=max_kv_bound or max_kv, captured=bool(max_kv_bound))
        notes = {}
        for sig, part in self._preparers.items():
            arrays, notes[sig] = part.prepare_step(batch)
            for name, values in arrays.items():
                chunks.append(np.asarray(values, dtype=i32).reshape(-1))
                layout.append(((sig, name), len(values)))
        group_layout = []
        for g in cache.groups:
            tables = [np.asarray(cache.table(g, e.request), dtype=i32) for e in entries]
            tables += [np.asarray([cache.scratch_page], dtype=i32)] * (S - n_real)
            width = table_width or max(1, max(len(t) for t in tables))
            padded = np.full((S, width), -1, dtype=i32)
            for row, t in zip(padded, tables):
                row[:len(t)] = t
            chunks.append(padded.reshape(-1))
            for t, where in zip(tables, positions):                   # where every new token's key and value go
                chunks.append(t[where // P] * P + where % P if len(where) else empty)
            group_layout.append((g, width))
        host = dict(seq_start=seq_start, seq_ctx=seq_ctx, seq_slots=seq_slots, n_logits=len(logit_rows),
                    max_q=max_q, max_kv=max_kv_bound or max_kv, notes=notes, T=T, S=S, captured=bool(max_kv_bound))
        return np.concatenate(chunks), layout, group_layout, host

    def _context_from(self, dev: torch.Tensor, layout, group_layout, host) -> StepContext:
        off = 0
        parts = {}
        for name, n in layout:
            parts[name] = dev[off:off + n]
            off += n
        T, S = host["T"], host["S"]
        block_tables, slot_maps = {}, {}
        for g, width in group_layout:
            block_tables[g] = dev[off:off + S * width].view(S, width)
            off += S * width
            slot_maps[g] = dev[off:off + T]
            off += T
        step_data = {sig: ({}, note) for sig, note in host["notes"].items()}
        for name in parts:
            if isinstance(name, tuple):
                step_data[name[0]][0][name[1]] = parts[name]
        return StepContext(
            rt=self.rt, n_tokens=T, n_seqs=S, token_ids=parts["token_ids"], positions=parts["positions"],
            row_seq=parts["row_seq"], seq_start=host["seq_start"], seq_ctx=host["seq_ctx"],
            seq_slots=host["seq_slots"], seq_start_dev=parts["seq_start"], seq_ctx_dev=parts["seq_ctx"],
            seq_slots_dev=parts["seq_slots"], logit_rows=parts["logit_rows"], n_logits=host["n_logits"],
            block_tables=block_tables, slot_maps=slot_maps, max_q_len=host["max_q"], max_kv_len=host["max_kv"],
            cache_views=self._views, step_data=step_data, captured=host["captured"])

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Host arrays of the batch, uploaded in one copy."""
        flat, layout, group_layout, host = self._host_arrays(entries)
        dev = torch.from_numpy(flat).to(self.rt.device, non_blocking=True)
        return self._context_from(dev, layout, group_layout, host)

    # ---- decode steps as captured graphs ------------------------------------------
    def _graph_eligible(self, entries: Sequence[StepEntry]) -> bool:
        return (self.use_graphs and len(entries) <= self.graph_max_batch
                and all(len(e.tokens) == 1 for e in entries))

    def graph_rows(self, n_requests: int) -> int:
        """Rows of the captured graph that serves a decode step of ``n_requests`` requests."""
        for rows in self.GRAPH_ROWS:
            if rows >= n_requests:
                return min(rows, max(self.graph_max_batch, n_requests))
        return n_requests

    def _graph_step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A step in which every request brings one token, replayed from a HIP graph captured
        for a number of rows (graph_rows: at least this step's) and a context bucket.  Only the int32
        batch description changes between replays; it is copied into the graph's own buffer first.
        Logits of the requests' rows come back ([requests, vocab]); the buffer is the graph's and is
        overwritten by its next replay."""
        cache, P = self.cache, self.cache.page_tokens
        n_real = len(entries)
        S = self.graph_rows(n_real)
        width = cache.max_pages_per_request
        slots = cache.slots([e.request for e in entries])
        if S > n_real:                      # the rows that stand for no request: the scratch slot, nothing cached
            slots = np.concatenate([slots, np.full(S - n_real, cache.scratch_slot, dtype=np.int32)])
        ctx = cache.lengths_by_slot[slots]
        bucket = 256
        while bucket < int(ctx.max()) + 1:
            bucket *= 2
        key = (S, bucket)
        slot = self._graphs.get(key)
        if slot is None:
            flat, layout, group_layout, host = self._host_arrays(entries, table_width=width, all_logits=True,
                                                                 max_kv_bound=bucket, pad_to=S)
            slot = self._capture(key, flat, layout, group_layout, host, bucket)
        else:
            self._graphs.move_to_end(key)
        # a ring of pinned staging buffers, each with an event that says its copy has been done
        ring = slot["ring"]
        buf, view, event = ring[slot["next"] % len(ring)]
        slot["next"] += 1
        event.synchronize()
        # What changes from step to step is written from the cache manager's arrays by slot, with no
        # loop over the requests; what does not (rows 0..S-1 one per request) is in the buffers since
        # the capture.  The layout is that of _host_arrays.
        at = slot["at"]
        view[0:n_real] = [e.tokens[0] for e in entries]
        view[at["positions"]:at["positions"] + S] = ctx
        view[at["seq_ctx"]:at["seq_ctx"] + S] = ctx
        view[at["seq_slots"]:at["seq_slots"] + S] = slots
        rows = slot["rows"]
        for g, tables_at, slots_at in at["groups"]:
            tables = cache.tables_by_slot[g][slots]
            view[tables_at:tables_at + S * width] = tables.reshape(-1)
            view[slots_at:slots_at + S] = tables[rows, ctx // P] * P + ctx % P
        if self._preparers:
            batch = HostBatch(n_tokens=S, n_seqs=S, seq_start=slot["seq_start"], seq_ctx=ctx, seq_slots=slots,
                              max_q_len=1, max_kv_len=bucket, captured=True)
            for sig, part in self._preparers.items():
                for name, values in part.prepare_step(batch)[0].items():
                    off, n = at[(sig, name)]
                    if len(values) != n:
                        raise EngineError(f"step: a captured step's array '{name}' of {type(part).__name__} changed its "
                                          f"length from {n} to {len(values)}")
                    view[off:off + n] = values
        slot["dev"].copy_(buf, non_blocking=True)
        event.record()
        if device_tokens is not None:
            slot["dev"][:n_real].copy_(device_tokens)
        slot["graph"].replay()
        return slot["logits"][:n_real]

    def _capture(self, key, flat, layout, group_layout, host, bucket):
        S = key[0]
        while len(self._graphs) >= self.MAX_GRAPHS:  # the graph used longest ago makes room (its memory goes with it)
            self._graphs.popitem(last=False)
        dev = torch.from_numpy(flat).to(self.rt.device)
        # Whatever the parts derive from the context is derived from the bucket's bound (host["max_kv"]), so
        # the launch geometry frozen into the graph holds for every context of the bucket.
        for part in self._capture_parts:
            part.prepare_capture(S, bucket)
        ctx = self._context_from(dev, layout, group_layout, host)
        self.model.forward(ctx)                      # once outside the graph: first-use work happens here
        torch.cuda.synchronize()
        ctx.made.clear()                             # what layers share is made again inside the graph
        graph = torch.cuda.CUDAGraph()
        # (thread_local: what another thread does on the device meanwhile -- the caller of an engine whose worker
        # runs this -- neither fails there nor spoils the capture)
        with torch.cuda.graph(graph, capture_error_mode="thread_local"):
            logits = self.model.forward(ctx)
        ring = []
        for _ in range(4):
            buf = torch.empty(len(flat), dtype=torch.int32).pin_memory()
            buf.numpy()[:] = flat
            event = torch.cuda.Event()
            event.record()
            ring.append((buf, buf.numpy(), event))
        # where the parts that change between steps lie in the flat array
        at, off = {}, 0
        for name, n in layout:
            at[name] = (off, n) if isinstance(name, tuple) else off
            off += n
        at["groups"] = []
        for g, width in group_layout:
            at["groups"].append((g, off, off + S * width))
            off += S * width + host["T"]
        slot = dict(graph=graph, dev=dev, logits=logits, ring=ring, next=0, at=at, rows=np.arange(S),
                    seq_start=list(range(S + 1)))
        self._graphs[key] = slot
        self.captures += 1
        return slot

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run the entries as one batch.  Returns float32 logits
        [number of wanted places, vocab] on the device, in the order of the
        entries and of their ``want`` lists; None if nothing is wanted.

        ``device_tokens`` (int32 on the device, one per entry): every entry brings one token, and it
        is this tensor's -- what a sampling kernel has just chosen -- not the placeholder in the
        entry.  The host can then describe the next step before it has seen the ids of this one,
        and read them while the next step runs.  The ids must lie in the vocabulary: they are not
        looked at on the host.

        Raises OutOfPages, with nothing changed, if the cache cannot hold the
        batch's tokens."""
        self._validate(entries)
        if device_tokens is not None:
            if (not device_tokens.is_cuda or device_tokens.dtype != torch.int32 or device_tokens.dim() != 1
                    or device_tokens.numel() != len(entries) or any(len(e.tokens) != 1 for e in entries)):
                raise EngineError("step: device_tokens must be int32 on the device, one for each entry, "
                                  "and every entry must bring one (placeholder) token")
        self.cache.reserve([(e.request, len(e.tokens)) for e in entries])
        if self._graph_eligible(entries):
            every = self._graph_step(entries, device_tokens)
            wanted = [i for i, e in enumerate(entries) if len(e.want)]
            if not wanted:
                logits = None
            elif len(wanted) == len(entries):
                logits = every
            else:
                logits = every[torch.tensor(wanted, device=every.device)]
        else:
            ctx = self.build_context(entries)
            if device_tokens is not None:
                ctx.token_ids.copy_(device_tokens)
            logits = self.model.forward(ctx)
        for e in entries:
            self.cache.advance(e.request, len(e.tokens))
        return logits
