"""The cache manager: pages of keys and values with a block table for each
request, and slots for per-request state of fixed size.

A model's cache *streams* (one per schedule entry that caches, or shared
between entries) each declare a spec, which says what it keeps and in which
tensors (see ``specs.py``; the manager knows no spec by name).  Streams that keep
something per token are put into *groups* by the rule under which their tokens may
be given back, which the spec states itself (``group_key``, ``first_kept``): all
streams that keep every token share one page pool and one block table per request;
streams with a window of W tokens share another, whose pages are given back once a
request's window has passed them.  Within a group one page index stands for the same
``page_tokens`` tokens in every stream of the group, each stream having tensors
of its own, ``[pages, *shape of one page]`` (for keys and values:
``[pages, kv_heads, page_tokens, head_dim]`` and, transposed,
``[pages, kv_heads, head_dim, page_tokens]``).
Streams that keep something per request get tensors ``[max_requests, *shape]``;
a request's row is its slot, zeroed at admission.

(Reference: KVCache, engine/include/llm/kv_cache.h:14-88 and
engine/src/kv_cache.cpp:17-153 -- one group, 64-token pages, one page table row
per slot, pages acquired lazily by reserve() and given back by reset().  Pages
are never cleared on reuse; masks never read past a request's length.)

The bookkeeping is host-side and does not touch the device except to zero a
state slot and, when asked, to poison pages.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Hashable, Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import EngineError, OutOfPages
from .page_pool import PagePool

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def _shape_and_dtype(entry, default: torch.dtype):
    """A spec names a tensor as a shape (in the cache's dtype) or as (shape, dtype name)."""
    if len(entry) == 2 and isinstance(entry[1], str):
        dt = _DTYPES.get(entry[1])
        if dt is None:
            raise EngineError(f"cache: dtype {entry[1]!r} is not one of {sorted(_DTYPES)}")
        return tuple(int(d) for d in entry[0]), dt
    return tuple(int(d) for d in entry), default


class View:
    """What a mixer sees of its cache stream: the stream's tensors by name (``view.k``, ``view.v``
    for keys and values; ``view.state`` for a state slot, row = request slot), and for a paged
    stream the key of the group whose block table addresses it, the page size and the window."""

    def __init__(self, tensors: Dict[str, torch.Tensor], group: Optional[Hashable] = None, page_tokens: int = 0,
                 window: int = 0):
        self.tensors = dict(tensors)
        self.group, self.page_tokens, self.window = group, page_tokens, window

    def __getattr__(self, name: str) -> torch.Tensor:
        try:
            return self.__dict__["tensors"][name]
        except KeyError:
            raise AttributeError(f"this cache stream has no tensor '{name}' (it has {sorted(self.__dict__.get('tensors', {}))})") from None

    @property
    def paged(self) -> bool:
        return self.group is not None


PagedView = StateView = View     # (the two kinds of view were classes of their own once)


def bytes_per_page(specs: Iterable[Any], page_tokens: int, dtype: torch.dtype) -> int:
    """Device bytes that one page index stands for, over all streams that keep something per token."""
    total = 0
    for spec in specs:
        if spec is not None and getattr(spec, "per_token", False):
            for entry in spec.page_tensors(page_tokens).values():
                shape, dt = _shape_and_dtype(entry, dtype)
                n = 1
                for d in shape:
                    n *= d
                total += n * torch.empty((), dtype=dt).element_size()
    return total


def _retention(spec):
    """(group key, first_kept, keeps everything) of a per-token spec: its own statement, or what its
    ``window`` says (0 or absent: every token is kept)."""
    window = int(getattr(spec, "window", 0))
    if hasattr(spec, "first_kept"):
        key = spec.group_key() if hasattr(spec, "group_key") else ("rule", type(spec).__name__, window)
        return key, spec.first_kept, key == ("window", 0)
    if window > 0:
        return ("window", window), (lambda length: max(0, length - window + 1)), False
    return ("window", 0), (lambda length: 0), True


class _Group:
    def __init__(self, window: int, num_pages: int, first_kept, keeps_all: bool):
        self.window = window                 # (what the views show; the rule itself is first_kept)
        self.first_kept = first_kept         # length -> earliest token still read by a query at `length` or later
        self.keeps_all = keeps_all
        self.pool = PagePool(num_pages)
        self.streams: List[Hashable] = []


class _Request:
    def __init__(self, slot: int, groups: Iterable[Hashable]):
        self.slot = slot
        self.length = 0
        # group -> page of every page index so far; -1 where the window has passed
        self.tables: Dict[Hashable, List[int]] = {g: [] for g in groups}
        self.released: Dict[Hashable, int] = {g: 0 for g in groups}  # leading pages given back


class CacheManager:
    def __init__(self, streams: Dict[Hashable, Any], *, page_tokens: int, num_pages: int,
                 max_requests: int, max_tokens: int, dtype: torch.dtype, device: Any,
                 poison: bool = False):
        if page_tokens <= 0 or num_pages < 0 or max_requests <= 0 or max_tokens <= 0:
            raise EngineError(f"cache: bad sizes page_tokens={page_tokens} num_pages={num_pages} "
                              f"max_requests={max_requests} max_tokens={max_tokens}")
        self.page_tokens = page_tokens
        self.max_requests = max_requests
        self.max_tokens = max_tokens
        self.max_pages_per_request = -(-max_tokens // page_tokens)
        self.dtype = dtype
        self.device = torch.device(device)
        self.poison = poison
        self.specs = dict(streams)
        self.groups: Dict[Hashable, _Group] = {}
        self._views: Dict[Hashable, Any] = {}
        for sid, spec in self.specs.items():
            if spec is None:
                continue
            if getattr(spec, "per_token", None) is True and hasattr(spec, "page_tensors"):
                window = int(getattr(spec, "window", 0))
                key, first_kept, keeps_all = _retention(spec)
                group = self.groups.get(key)
                if group is None:
                    group = self.groups[key] = _Group(window, num_pages, first_kept, keeps_all)
                group.streams.append(sid)
                tensors = {}
                for name, entry in spec.page_tensors(page_tokens).items():
                    shape, dt = _shape_and_dtype(entry, dtype)
                    t = torch.empty((num_pages + 1, *shape), dtype=dt, device=self.device)   # (+ the scratch page)
                    if poison and t.is_floating_point():
                        t.fill_(float("nan"))
                    tensors[name] = t
                self._views[sid] = View(tensors, group=key, page_tokens=page_tokens, window=window)
            elif getattr(spec, "per_token", None) is False and hasattr(spec, "slot_tensors"):
                tensors = {}
                for name, entry in spec.slot_tensors().items():
                    shape, dt = _shape_and_dtype(entry, dtype)
                    tensors[name] = torch.zeros((max_requests + 1, *shape), dtype=dt, device=self.device)  # (+ the scratch slot)
                self._views[sid] = View(tensors)
            else:
                raise EngineError(f"cache: stream {sid!r} has a spec that says neither what it keeps per token "
                                  f"(per_token = True, page_tensors) nor per request (per_token = False, slot_tensors): {spec!r}")
        self._requests: Dict[Hashable, _Request] = {}
        self._peaks: Dict[Tuple[int, int], Dict[Hashable, int]] = {}
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        # The same bookkeeping as arrays by request slot, for whoever describes a batch of many
        # requests to the device without a Python loop over them: lengths, and every group's block
        # tables as rows of a matrix (-1 where there is no page), kept in step with the lists above.
        # One page and one slot beyond those that requests can hold: the *scratch* page (index num_pages, in no
        # pool) and the scratch slot (index max_requests, never admitted to).  Rows that stand for no request --
        # the rows that fill a captured decode step up to its graph's size -- write their keys and their state
        # there and read nothing else.  The arrays by slot have a row for it: no tokens, one page.
        self.scratch_page, self.scratch_slot = num_pages, max_requests
        self.lengths_by_slot = np.zeros(max_requests + 1, dtype=np.int32)
        self.tables_by_slot: Dict[Hashable, np.ndarray] = {
            g: np.full((max_requests + 1, self.max_pages_per_request), -1, dtype=np.int32) for g in self.groups}
        for t in self.tables_by_slot.values():
            t[self.scratch_slot, 0] = self.scratch_page

    # ---- requests ---------------------------------------------------------
    def has(self, request: Hashable) -> bool:
        return request in self._requests

    def live_requests(self) -> List[Hashable]:
        return list(self._requests)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, request: Hashable) -> int:
        """Give the request a slot (zeroing its state); returns the slot."""
        if request in self._requests:
            raise EngineError(f"cache: request {request!r} is already live")
        if not self._free_slots:
            raise EngineError(f"cache: all {self.max_requests} request slots are taken")
        slot = self._free_slots.pop()
        self._requests[request] = _Request(slot, self.groups)
        self.lengths_by_slot[slot] = 0
        for view in self._views.values():
            if not view.paged:
                for t in view.tensors.values():
                    t[slot].zero_()
        return slot

    def _req(self, request: Hashable) -> _Request:
        try:
            return self._requests[request]
        except KeyError:
            raise EngineError(f"cache: unknown request {request!r}") from None

    def slot(self, request: Hashable) -> int:
        return self._req(request).slot

    def length(self, request: Hashable) -> int:
        return self._req(request).length

    def slots(self, requests: Sequence[Hashable]) -> np.ndarray:
        """The requests' slots as an array: the index into lengths_by_slot and tables_by_slot."""
        try:
            return np.fromiter((self._requests[r].slot for r in requests), dtype=np.int32, count=len(requests))
        except KeyError as e:
            raise EngineError(f"cache: unknown request {e.args[0]!r}") from None

    def table(self, group: Hashable, request: Hashable) -> List[int]:
        """The request's pages in token order (-1 where the window has passed)."""
        return self._req(request).tables[group]

    # ---- pages ------------------------------------------------------------
    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_tokens)

    def new_pages_needed(self, request: Hashable, n_new: int) -> Dict[Hashable, int]:
        r = self._req(request)
        want = self.pages_for(r.length + n_new)
        return {g: max(0, want - len(t)) for g, t in r.tables.items()}

    def can_reserve(self, asks: Sequence[Tuple[Hashable, int]]) -> bool:
        need: Dict[Hashable, int] = {g: 0 for g in self.groups}
        for request, n_new in asks:
            for g, n in self.new_pages_needed(request, n_new).items():
                need[g] += n
        return all(need[g] <= self.groups[g].pool.free_count for g in need)

    def reserve(self, asks: Sequence[Tuple[Hashable, int]]) -> None:
        """Make sure every (request, n_new) has pages for its next n_new tokens.

        All or nothing: if any group lacks pages, OutOfPages is raised and no
        page has been taken.  A request may appear once.
        """
        seen = set()
        need: Dict[Hashable, int] = {g: 0 for g in self.groups}
        short = False
        for request, n_new in asks:
            if request in seen:
                raise EngineError(f"cache: request {request!r} appears twice in one reservation")
            seen.add(request)
            r = self._req(request)
            if n_new < 0:
                raise EngineError(f"cache: negative token count {n_new} for request {request!r}")
            if r.length + n_new > self.max_tokens:
                raise EngineError(f"cache: request {request!r} would hold {r.length + n_new} tokens, "
                                  f"the cache is sized for {self.max_tokens} per request")
            want = -(-(r.length + n_new) // self.page_tokens)
            for g, t in r.tables.items():
                if len(t) < want:
                    need[g] += want - len(t)
                    short = True
        if not short:
            return
        for g, n in need.items():
            free = self.groups[g].pool.free_count
            if n > free:
                raise OutOfPages(f"out of pages: group {g} needs {n} more, {free} of "
                                 f"{self.groups[g].pool.num_pages} are free")
        for request, n_new in asks:
            r = self._requests[request]
            want = self.pages_for(r.length + n_new)
            for g, t in r.tables.items():
                while len(t) < want:
                    page = self.groups[g].pool.acquire()
                    assert page >= 0
                    self.tables_by_slot[g][r.slot, len(t)] = page
                    t.append(page)

    def advance(self, request: Hashable, n_new: int) -> None:
        """The request's next n_new tokens are now cached.  Pages that every
        later query's window has passed go back to their pool."""
        r = self._req(request)
        if n_new < 0 or (r.tables and
                         r.length + n_new > min(len(t) for t in r.tables.values()) * self.page_tokens):
            raise EngineError(f"cache: request {request!r} advanced past its reserved pages")
        r.length += n_new
        self.lengths_by_slot[r.slot] = r.length
        for g, t in r.tables.items():
            group = self.groups[g]
            if group.keeps_all:
                continue
            # the next query sits at position r.length; pages wholly before what it and later ones read go back
            first_needed = max(0, int(group.first_kept(r.length))) // self.page_tokens
            for idx in range(r.released[g], min(first_needed, len(t))):
                self._give_back(g, t[idx])
                t[idx] = -1
                self.tables_by_slot[g][r.slot, idx] = -1
            r.released[g] = max(r.released[g], min(first_needed, len(t)))

    def _give_back(self, group: Hashable, page: int) -> None:
        if not self.groups[group].pool.release(page):
            raise EngineError(f"cache: page {page} of group {group} was freed twice or never held")
        if self.poison:
            for sid in self.groups[group].streams:
                for t in self._views[sid].tensors.values():
                    if t.is_floating_point():
                        t[page].fill_(float("nan"))

    def release(self, request: Hashable) -> None:
        """The request has ended: its pages and its slot are given back."""
        r = self._req(request)
        for g, t in r.tables.items():
            for page in t:
                if page >= 0:
                    self._give_back(g, page)
            self.tables_by_slot[g][r.slot, :len(t)] = -1
        self.lengths_by_slot[r.slot] = 0
        self._free_slots.append(r.slot)
        del self._requests[request]

    def peak_pages(self, total_tokens: int, portion: int) -> Dict[Hashable, int]:
        """group -> the most pages one request holds at a time while ``total_tokens`` tokens are fed
        to it in portions of at most ``portion``, however they are cut: a step that begins at length p
        holds the pages from first_kept(p) to p + its tokens.  Nothing for a model whose streams keep
        nothing per token."""
        key = (total_tokens, portion)
        hit = self._peaks.get(key)
        if hit is not None:
            return hit
        P, out = self.page_tokens, {}
        for g, group in self.groups.items():
            if group.keeps_all:
                out[g] = -(-total_tokens // P)
                continue
            most = 0
            for p in range(0, max(total_tokens, 1)):
                upto = min(p + max(portion, 1), total_tokens)
                most = max(most, -(-upto // P) - max(0, int(group.first_kept(p))) // P)
            out[g] = most
        if len(self._peaks) > 4096:
            self._peaks.clear()
        self._peaks[key] = out
        return out

    def release_all(self) -> None:
        for request in list(self._requests):
            self.release(request)

    # ---- views and numbers ---------------------------------------------------
    def view(self, stream: Hashable):
        return self._views.get(stream)

    def pages_in_use(self, group: Optional[Hashable] = None) -> int:
        if group is not None:
            return self.groups[group].pool.pages_in_use
        return sum(g.pool.pages_in_use for g in self.groups.values())

    def pages_total(self) -> int:
        return sum(g.pool.num_pages for g in self.groups.values())

    def free_pages(self, group: Hashable) -> int:
        return self.groups[group].pool.free_count

    def shuffle_free_pages(self, seed: int) -> None:
        for i, g in enumerate(self.groups.values()):
            g.pool.shuffle_free_list(seed + i)

    def storage_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for view in self._views.values() for t in view.tensors.values())
