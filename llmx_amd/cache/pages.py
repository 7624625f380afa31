"""Page ids and per-request state slots: the logical side of the cache, host only.

The pool hands out ids dense from zero, reuses the most recently freed id first, counts references, and refuses a
double release, a retain of a free page and an empty pool (/root/reference/src/model/kv_cache.hpp:14-67).
"""

from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """The pool cannot give the pages a step needs."""


class CacheLogicError(RuntimeError):
    """A misuse of the cache manager (double release, unknown request, ...)."""


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages < 0:
            raise ValueError("a pool cannot hold a negative number of pages")
        self.capacity = int(n_pages)
        self._next = 0
        self._free: List[int] = []
        self._refs: List[int] = []

    def alloc(self) -> int:
        if self._free:
            page = self._free.pop()
            self._refs[page] = 1
            return page
        if self._next >= self.capacity:
            raise OutOfPages("cache: page budget exhausted; the run needs more tokens than the cache was made for")
        self._refs.append(1)
        self._next += 1
        return self._next - 1

    def retain(self, page: int) -> None:
        if not 0 <= page < self._next or self._refs[page] == 0:
            raise CacheLogicError(f"cache: retain of free page {page}")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        if not 0 <= page < self._next or self._refs[page] == 0:
            raise CacheLogicError(f"cache: page {page} released twice")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refs(self, page: int) -> int:
        return self._refs[page] if 0 <= page < self._next else 0

    @property
    def in_use(self) -> int:
        return self._next - len(self._free)

    @property
    def available(self) -> int:
        return self.capacity - self.in_use


class StateSlots:
    """Slots of fixed size, one per live request; the slot number indexes every per-request device array."""

    def __init__(self, n_slots: int):
        self.capacity = int(n_slots)
        self._free = list(range(self.capacity - 1, -1, -1))
        self._held = [False] * self.capacity

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("cache: every request slot is taken")
        slot = self._free.pop()
        self._held[slot] = True
        return slot

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.capacity or not self._held[slot]:
            raise CacheLogicError(f"cache: slot {slot} released twice")
        self._held[slot] = False
        self._free.append(slot)

    @property
    def in_use(self) -> int:
        return self.capacity - len(self._free)
