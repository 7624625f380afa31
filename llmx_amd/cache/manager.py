"""The cache manager: for every live request a state slot and, in every cache group, a table of pages.

Layers with the same need (kv heads, head width, all keys or a window of them) form a group with a pool of its own.
A step first reserves (`prepare`) the pages its rows will write, in every group or in none; after the step ran it
commits, which also gives back the pages of a windowed group that no later row can read; a failed step aborts and
returns exactly the pages the attempt took (/root/reference/src/model/kv_cache.hpp:71-179).  `truncate` takes a request
back to a shorter length and returns the pages beyond it (:126-134).  Ending a request gives everything back.

State slots and a failing step: with `shadow_slots` a step writes each request's fixed-size state into a second slot
(the engine copies the live state there first); commit makes that slot the request's and frees the old one, abort frees
the second slot and the live state is as the step found it (the reference keeps the live slot as a mark while the next
pass writes another: kv_cache.hpp:216-266).
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

    def pool_pages(self, total_tokens: int, requests: int, step_tokens: Optional[int]) -> int:
        """Pages of a pool made for `total_tokens` tokens: all of them for a group that keeps every key; for a window,
        when the most tokens a step brings of one request is known, what `requests` requests can hold at once."""
        whole = self.pages_for(total_tokens)
        if self.window is None or step_tokens is None:
            return whole
        return min(whole, requests * self.peak_pages(total_tokens, step_tokens))


@dataclass
class _Request:
    slot: int
    length: int = 0
    pending: int = 0
    shadow: int = -1          # the slot the pending step writes its state to (-1: none, the step writes `slot`)
    tables: List[List[int]] = field(default_factory=list)   # per group: page of block i, -1 once given back
    taken: List[List[int]] = field(default_factory=list)    # per group: block indices the pending step allocated


class CacheManager:
    def __init__(self, groups: List[GroupSpec], max_requests: int, shadow_slots: bool = False):
        self.groups = list(groups)
        self.pools = [PagePool(g.n_pages) for g in self.groups]
        self.max_requests = int(max_requests)
        self.shadow_slots = bool(shadow_slots)
        # with shadows every live request may hold a second slot while its step runs
        self.slots = StateSlots(self.max_requests * (2 if self.shadow_slots else 1))
        self._requests: Dict[Hashable, _Request] = {}

    # -- requests -------------------------------------------------------------
    def open(self, request: Hashable) -> int:
        if request in self._requests:
            raise CacheLogicError(f"cache: request {request!r} is already open")
        if len(self._requests) >= self.max_requests:
            raise OutOfPages("cache: every request slot is taken")
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
        """The slot that holds the request's committed state."""
        return self._get(request).slot

    def step_slot(self, request: Hashable) -> int:
        """The slot the request's pending step reads and writes: its shadow when it has one, else its own."""
        r = self._get(request)
        return r.shadow if r.shadow >= 0 else r.slot

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
            if self.shadow_slots:
                r.shadow = self.slots.alloc()
        except OutOfPages:
            self._return_taken(r)
            raise
        r.pending = n

    def commit(self, request: Hashable) -> None:
        r = self._get(request)
        r.length += r.pending
        r.pending = 0
        if r.shadow >= 0:       # what the step wrote becomes the request's state
            self.slots.release(r.slot)
            r.slot, r.shadow = r.shadow, -1
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
        if r.shadow >= 0:       # the live state was never written
            self.slots.release(r.shadow)
            r.shadow = -1

    def truncate(self, request: Hashable, length: int) -> None:
        """Takes the request back to its first `length` tokens: the pages beyond them go back to their pools, in every
        group.  Refused (nothing changes) during a step, for a length above the present one, and when a windowed
        group has already given back a page that a row at position `length` would read."""
        r = self._get(request)
        if r.pending:
            raise CacheLogicError(f"cache: request {request!r} has a step in progress")
        if not 0 <= length <= r.length:
            raise CacheLogicError(f"cache: request {request!r} holds {r.length} tokens and cannot be taken back to {length}")
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            table = r.tables[gi]
            first = max(0, length - g.window + 1)     # the row at `length` reads keys first .. length - 1
            for i in range(first // g.page_tokens, g.pages_for(length)):
                if table[i] < 0:
                    raise CacheLogicError(f"cache: request {request!r} cannot be taken back to {length} tokens: {g.name} keeps the last "
                                          f"{g.window} keys only and has given back the page of position {i * g.page_tokens}")
        for gi, g in enumerate(self.groups):
            table = r.tables[gi]
            keep = g.pages_for(length)
            while len(table) > keep:
                page = table.pop()
                if page >= 0:
                    self.pools[gi].release(page)
        r.length = length

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
        if r.shadow >= 0:
            self.slots.release(r.shadow)
        del self._requests[request]

    # -- accounting -----------------------------------------------------------
    def pages_in_use(self, group: int = 0) -> int:
        return self.pools[group].in_use

    def pages_available(self, group: int = 0) -> int:
        return self.pools[group].available

    def pages_held(self, request: Hashable, group: int = 0) -> int:
        return sum(1 for p in self._get(request).tables[group] if p >= 0)
