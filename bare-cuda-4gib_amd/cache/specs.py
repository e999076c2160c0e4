"""What a mixer asks of the cache manager.

A cache spec says what is kept and in which tensors; the manager allocates them and does the
bookkeeping, and knows no spec by name.  Two kinds:

per token   ``per_token = True``.  ``page_tensors(page_tokens)`` names the tensors of ONE page
            (name -> shape, or name -> (shape, dtype name) for a tensor that is not in the cache's
            own dtype); the manager allocates ``[num_pages, *shape]`` of each.  When its tokens may be
            given back the spec says itself: ``first_kept(length)`` is the earliest token that any
            query at position ``length`` or later still reads (0: every token is kept), and pages
            wholly before it go back to their pool; ``group_key()`` names the rule -- specs with equal
            keys share a page pool and one block table per request.  A spec that has neither is read
            by its ``window`` (0 or absent = keep everything; W = a query reads the W tokens up to and
            including its own).
per request ``per_token = False``.  ``slot_tensors()`` names the tensors of ONE request slot
            (name -> (shape, dtype name)); the manager allocates ``[max_requests, *shape]`` of each and
            zeroes a slot when a request is admitted to it.

A mixer gets a :class:`View` of its stream: the tensors by name (``view.k``, ``view.state``, ...) and,
for a paged stream, ``group`` (the key of its block table and slot map in the step's context),
``page_tokens`` and ``window``.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Tuple


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values per token, in pages.  ``window`` 0 keeps every token;
    otherwise only the last ``window`` tokens are ever read again, and pages
    that a request's window has passed are given back.  Keys lie
    ``[page, kv_head, token, dim]``, values transposed ``[page, kv_head, dim, token]``
    (consecutive tokens of one dimension lie together)."""
    num_kv_heads: int
    head_dim: int
    window: int = 0
    per_token = True

    def page_tensors(self, page_tokens: int) -> Dict[str, Tuple[int, ...]]:
        return {"k": (self.num_kv_heads, page_tokens, self.head_dim),
                "v": (self.num_kv_heads, self.head_dim, page_tokens)}

    def group_key(self):
        return ("window", self.window)

    def first_kept(self, length: int) -> int:
        """The query at position ``length`` reads keys from ``length - window + 1`` on."""
        return max(0, length - self.window + 1) if self.window > 0 else 0


@dataclasses.dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (any shape), zeroed when the request is
    admitted, kept across its steps, dropped when it ends."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
    per_token = False

    def slot_tensors(self) -> Dict[str, Tuple[Tuple[int, ...], str]]:
        return {"state": (tuple(self.shape), self.dtype)}
