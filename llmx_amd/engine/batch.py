"""One step's rows as the parts see them: the row plan on the device and scratch storage.

The row plan follows the reference's `begin` (/root/reference/src/model/passes.hpp:369-392): token ids, positions that
continue each request's length, the rows whose logits are wanted; it is uploaded in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Sequence, Tuple

import numpy as np
import torch

from ..limits import MAX_STEP_ROWS


@dataclass(frozen=True)
class StepEntry:
    """A request's next tokens in a step, and the places among them whose logits are wanted."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass(frozen=True)
class EntryView:
    request: Hashable
    slot: int      # the request's state slot
    row0: int      # its first row in the step
    n: int         # its number of rows
    past: int      # tokens it held before the step


class StepError(ValueError):
    """A batch the step function refuses; nothing was reserved or run."""


def check_entries(entries: Sequence[StepEntry], cache, max_positions: int, vocab: int) -> List[EntryView]:
    """The refusals that come before anything is reserved (/root/reference/src/model/passes.hpp:271-413): an empty
    batch, a request named twice or not open, an entry without tokens, a context that would be exceeded, a token id
    outside the embedding's rows, a wanted place outside the entry, more rows than a step takes.  Returns the entries'
    views (slot, first row, rows, tokens held before)."""
    if not entries:
        raise StepError("step: an empty batch")
    seen = set()
    views: List[EntryView] = []
    row0 = 0
    for e in entries:
        if e.request in seen:
            raise StepError(f"step: request {e.request!r} appears twice in one batch")
        seen.add(e.request)
        if not cache.is_open(e.request):
            raise StepError(f"step: request {e.request!r} is not open")
        n = len(e.tokens)
        if n == 0:
            raise StepError(f"step: request {e.request!r} brings no tokens")
        past = cache.length(e.request)
        if past + n > max_positions:
            raise StepError(f"step: context length exceeded: request {e.request!r} would hold {past + n} tokens of {max_positions}")
        for t in e.tokens:
            if not 0 <= int(t) < vocab:
                raise StepError(f"step: token id {t} is outside the embedding's rows")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise StepError(f"step: request {e.request!r} wants the logits of place {w} among {n} tokens")
        views.append(EntryView(e.request, cache.slot(e.request), row0, n, past))
        row0 += n
    if row0 > MAX_STEP_ROWS:
        raise StepError(f"step: {row0} token rows in one step; a step takes at most {MAX_STEP_ROWS}")
    return views


class Workspace:
    """Scratch tensors by name; a name keeps its storage and grows when a larger shape is asked for."""

    def __init__(self, device: torch.device):
        self.device = device
        self._store: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self.generation = 0     # counts allocations: addresses handed out before a change may be stale

    def get(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        count = 1
        for d in shape:
            count *= int(d)
        key = (name, dtype)
        flat = self._store.get(key)
        if flat is None or flat.numel() < count:
            flat = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._store[key] = flat
            self.generation += 1
        return flat[:count].view(*shape)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._store.values())


class StepState:
    """What the parts read of a step (see parts/base.py for the interface)."""

    def __init__(self, workspace: Workspace, act_dtype: torch.dtype):
        self._ws = workspace
        self.act_dtype = act_dtype
        self.device = workspace.device
        self.rows = 0
        self.entries: List[EntryView] = []
        self.token_ids = self.positions = self.row_entry = self.entry_slots = self.pick = None
        self._tables: List[torch.Tensor] = []
        self.max_rows_per_entry = 0
        self._shared: Dict = {}
        self.run_index = -1          # which item of the run order is running
        self.observer = None         # callable(step, kind, **tensors) that sees what parts choose to show, or None

    def buf(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        return self._ws.get(name, shape, dtype)

    def tables(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def shared(self, key, make):
        """Something a part wants once a step: `make()` is called at the key's first use in this step; every later use
        (another layer with the same sizes) gets the same object.  A kernel's work plan for the step's rows, a second
        stream of positions, anything that depends on the step and not on the layer."""
        try:
            return self._shared[key]
        except KeyError:
            value = self._shared[key] = make()
            return value

    def observe(self, kind: str, **tensors) -> None:
        """Shows intermediate tensors (a router's picks, for instance) to the engine's observer, when one is set."""
        if self.observer is not None:
            self.observer(self, kind, **tensors)


class RowPlanUploader:
    """Packs the row plan into one pinned int32 buffer and copies it to the device once."""

    def __init__(self, device: torch.device):
        self.device = device
        self._host = None
        self._dev = None
        self._done = None
        self.generation = 0     # counts allocations of the device buffer

    def upload(self, arrays: List[np.ndarray]) -> List[torch.Tensor]:
        total = sum(a.size for a in arrays)
        if self._host is None or self._host.numel() < total:
            cap = max(1024, 2 * total)
            self._host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._done = None
            self.generation += 1
        if self._done is not None:
            self._done.synchronize()  # the previous copy has left the pinned buffer
        host = self._host.numpy()
        at = 0
        views = []
        for a in arrays:
            host[at:at + a.size] = a.reshape(-1)
            views.append(self._dev[at:at + a.size].view(*a.shape))
            at += a.size
        self._dev[:total].copy_(self._host[:total], non_blocking=True)
        self.mark()
        return views

    def mark(self) -> None:
        """Everything enqueued so far (the copy, kernels that read the device buffer) must end before the pinned buffer
        and the device buffer are written again."""
        self._done = torch.cuda.Event()
        self._done.record()
