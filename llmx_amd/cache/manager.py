"""The cache manager: for every live request a state slot and, in every cache group, a table of pages.

Layers with the same need (kv heads, head width, all keys or a window of them) form a group with a pool of its own.
A step first reserves (`prepare`) the pages its rows will write, in every group or in none; after the step ran it
commits, which also gives back the pages of a windowed group that no later row can read; a failed step aborts and
returns exactly the pages the attempt took (/root/reference/src/model/kv_cache.hpp:71-179).  Ending a request gives
everything back.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional

from .pages import CacheLogicError, OutOfPages, PagePool, StateSlots


@dataclass(frozen=True)
class GroupSpec:
    name: str
    page_tokens: int
    n_pages: int
    window: Optional[int] = None  # None: every key is kept; w: a row at p reads keys p-w+1 .. p

    def pages_for(self, tokens: int) -> int:
        return -(-tokens // self.page_tokens)

    def peak_pages(self, total_tokens: int, step_tokens: int) -> int:
        """Most pages a request of `total_tokens` holds at once when a step brings at most `step_tokens` of its tokens."""
        whole = self.pages_for(total_tokens)
        if self.window is None:
            return whole
        return min(whole, self.pages_for(self.window + step_tokens) + 1)


@dataclass
class _Request:
    slot: int
    length: int = 0
    pending: int = 0
    tables: List[List[int]] = field(default_factory=list)   # per group: page of block i, -1 once given back
    taken: List[List[int]] = field(default_factory=list)    # per group: block indices the pending step allocated


class CacheManager:
    def __init__(self, groups: List[GroupSpec], max_requests: int):
        self.groups = list(groups)
        self.pools = [PagePool(g.n_pages) for g in self.groups]
        self.slots = StateSlots(max_requests)
        self._requests: Dict[Hashable, _Request] = {}

    # -- requests -------------------------------------------------------------
    def open(self, request: Hashable) -> int:
        if request in self._requests:
            raise CacheLogicError(f"cache: request {request!r} is already open")
        slot = self.slots.alloc()
        self._requests[request] = _Request(slot, tables=[[] for _ in self.groups], taken=[[] for _ in self.groups])
        return slot

    def is_open(self, request: Hashable) -> bool:
        return request in self._requests

    def _get(self, request: Hashable) -> _Request:
        try:
            return self._requests[request]
        except KeyError:
            raise CacheLogicError(f"cache: request {request!r} is not open") from None

    def slot(self, request: Hashable) -> int:
        return self._get(request).slot

    def length(self, request: Hashable) -> int:
        return self._get(request).length

    def table(self, request: Hashable, group: int) -> List[int]:
        return self._get(request).tables[group]

    def live(self) -> List[Hashable]:
        return list(self._requests)

    # -- a step's transaction ---------------------------------------------------
    def prepare(self, request: Hashable, n: int) -> None:
        """Make positions [length, length+n) writable in every group, or change nothing and raise OutOfPages."""
        r = self._get(request)
        if r.pending:
            raise CacheLogicError(f"cache: request {request!r} already has a step in progress")
        if n <= 0:
            raise CacheLogicError("cache: a step brings at least one token")
        try:
            for gi, g in enumerate(self.groups):
                need = g.pages_for(r.length + n)
                table = r.tables[gi]
                while len(table) < need:
                    table.append(self.pools[gi].alloc())
                    r.taken[gi].append(len(table) - 1)
        except OutOfPages:
            self._return_taken(r)
            raise
        r.pending = n

    def commit(self, request: Hashable) -> None:
        r = self._get(request)
        r.length += r.pending
        r.pending = 0
        for gi, g in enumerate(self.groups):
            r.taken[gi].clear()
            if g.window is not None:
                # the next row sits at position >= length and reads keys >= length - window + 1
                dead_below = r.length - g.window + 1
                table = r.tables[gi]
                for i in range(len(table)):
                    if (i + 1) * g.page_tokens > dead_below:
                        break
                    if table[i] >= 0:
                        self.pools[gi].release(table[i])
                        table[i] = -1

    def abort(self, request: Hashable) -> None:
        r = self._get(request)
        self._return_taken(r)
        r.pending = 0

    def _return_taken(self, r: _Request) -> None:
        for gi in range(len(self.groups)):
            table = r.tables[gi]
            for i in reversed(r.taken[gi]):
                self.pools[gi].release(table[i])
                assert i == len(table) - 1
                table.pop()
            r.taken[gi].clear()

    def close(self, request: Hashable) -> None:
        """The request ended: every page and the slot go back."""
        r = self._get(request)
        for gi in range(len(self.groups)):
            for page in reversed(r.tables[gi]):
                if page >= 0:
                    self.pools[gi].release(page)
        self.slots.release(r.slot)
        del self._requests[request]

    # -- accounting -----------------------------------------------------------
    def pages_in_use(self, group: int = 0) -> int:
        return self.pools[group].in_use

    def pages_available(self, group: int = 0) -> int:
        return self.pools[group].available

    def pages_held(self, request: Hashable, group: int = 0) -> int:
        return sum(1 for p in self._get(request).tables[group] if p >= 0)
