"""Allocators of page ids and of state slots.

``PageAllocator`` follows the contract of the reference's ``GlobalKvAllocator``
(crates/infer-worker/src/domain/global_kv_alloc.rs:56-380): ``alloc(n)`` hands out the
``n`` smallest free ids in ascending order, so block tables, and with them a replay, are
the same for the same history; ``free`` makes ids allocatable at once.  It is stricter
in one point: freeing an id that is not held is an error here, not a warning, because
this engine has one owner of every page.
"""
from __future__ import annotations

import heapq
from typing import Iterable, List


class CacheError(RuntimeError):
    """Misuse of the cache manager (double free, unknown request, ...)."""


class OutOfPages(CacheError):
    """Not enough free pages (or slots): the caller decides who waits or is preempted.
    Mirrors ``AllocFull{need, available}`` (global_kv_alloc.rs:34-40)."""

    def __init__(self, need: int, available: int, what: str = "pages"):
        super().__init__(f"out of {what}: need {need}, {available} free")
        self.need, self.available, self.what = need, available, what


class PageAllocator:
    def __init__(self, total: int, what: str = "pages"):
        if total < 0:
            raise ValueError("total must be >= 0")
        self.total = int(total)
        self.what = what
        self._free: List[int] = list(range(self.total))   # already a valid heap
        self._held = bytearray(self.total)                 # 1 = handed out

    @property
    def available(self) -> int:
        return len(self._free)

    @property
    def outstanding(self) -> int:
        return self.total - len(self._free)

    def alloc(self, n: int) -> List[int]:
        if n < 0:
            raise ValueError("n must be >= 0")
        if n > len(self._free):
            raise OutOfPages(n, len(self._free), self.what)
        out = [heapq.heappop(self._free) for _ in range(n)]
        for i in out:
            self._held[i] = 1
        return out

    def free(self, ids: Iterable[int]) -> None:
        ids = list(ids)
        seen = set()
        for i in ids:
            if not (0 <= i < self.total):
                raise CacheError(f"free of {self.what[:-1]} {i} outside [0, {self.total})")
            if i in seen or not self._held[i]:
                raise CacheError(f"{self.what[:-1]} {i} freed twice")
            seen.add(i)
        for i in ids:
            self._held[i] = 0
            heapq.heappush(self._free, i)

    def is_held(self, i: int) -> bool:
        return bool(self._held[i])
