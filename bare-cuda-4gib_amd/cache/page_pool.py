"""A pool of fixed-size pages identified by index.

Same contract as the reference's PagePool (engine/src/allocator.cpp:18-65,
engine/include/llm/allocator.h:12-45): a LIFO free list filled so that a fresh
pool hands out 0, 1, 2, ...; ``acquire`` returns -1 when empty; ``release``
refuses an invalid index or a page that is not in use; a high-water mark; and
``shuffle_free_list`` so tests can scatter pages.  The pool only counts: the
memory the indices stand for belongs to the cache manager.
"""
from __future__ import annotations

import random
from typing import List


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError(f"num_pages must not be negative, got {num_pages}")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() gives 0 first
        self._in_use = [False] * num_pages
        self._used = 0
        self.high_water_mark = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def pages_in_use(self) -> int:
        return self._used

    def in_use(self, page: int) -> bool:
        return 0 <= page < self.num_pages and self._in_use[page]

    def acquire(self) -> int:
        if not self._free:
            return -1
        page = self._free.pop()
        self._in_use[page] = True
        self._used += 1
        self.high_water_mark = max(self.high_water_mark, self._used)
        return page

    def release(self, page: int) -> bool:
        if not (0 <= page < self.num_pages) or not self._in_use[page]:
            return False
        self._in_use[page] = False
        self._used -= 1
        self._free.append(page)
        return True

    def shuffle_free_list(self, seed: int) -> None:
        random.Random(seed).shuffle(self._free)
