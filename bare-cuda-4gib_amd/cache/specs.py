"""What a mixer asks of the cache manager."""
from __future__ import annotations

import dataclasses
from typing import Tuple


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values per token, in pages.  ``window`` 0 keeps every token;
    otherwise only the last ``window`` tokens are ever read again, and pages
    that a request's window has passed are given back."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclasses.dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (any shape), zeroed when the request is
    admitted, kept across its steps, dropped when it ends."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
