"""Interfaces of the parts a layer is made of, and the registries that map a part's name to its class.

A part is built from its parameters alone (`PartSpec.params`), says which tensors it reads (`tensor_specs`), takes
them (`load`), and runs on the rows of one step.  No part knows which model it is in.

What a part sees of a step (the `step` argument, an `engine.batch.StepState`):
  step.rows                       number of token rows T in this step
  step.act_dtype                  torch.float32 or torch.bfloat16: the type products read their inputs in
  step.token_ids, step.positions  int32 [T] on the device
  step.row_entry                  int32 [T]: index of each row's request among the step's entries
  step.entries                    host list of EntryView(slot, row0, n, past): a request's state slot, its first row,
                                  its number of rows and the tokens it held before the step
  step.entry_slots                int32 [n_entries] on the device: each entry's state slot
  step.tables(group)              int32 [n_entries, max_blocks]: page ids of each entry in cache group `group`
  step.buf(name, shape, dtype)    a scratch tensor that lives until the step ends (same name, same storage)
  step.shared(key, make)          something a part wants once a step (a kernel's work plan, a second position stream):
                                  make() is called at the key's first use in the step, later uses get the same object
  step.run_index                  which item of the run order is running
  step.observe(kind, **tensors)   shows intermediate tensors to an observer, when the engine has one (tests, probes)
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Set, Union

import torch

from .spec import PagedNeed, PartSpec, StateNeed, TensorSpec


@dataclass
class BuildContext:
    """What a part needs to know of the engine it is built into."""
    act_dtype: torch.dtype        # float32: the true 32-bit path; bfloat16: the serving path
    device: torch.device
    max_positions: int            # positions the engine can reach (context or the cache's tokens, whichever is smaller)
    page_tokens: Optional[int] = None   # tokens a cache page holds (None where no cache is made: listing tensors)

    @property
    def exact(self) -> bool:
        return self.act_dtype == torch.float32


class Part:
    """Base of every part."""

    kind: str = ""
    #: True when `forward` only launches this package's kernels on the current stream into storage from `step.buf`
    #: (no allocation, no host synchronisation, no library call that could record a fill into a captured graph);
    #: the engine replays decode steps as HIP graphs only if every part of the model says so.
    graph_safe: bool = False

    def __init__(self, params: dict, prefix: str, ctx: BuildContext):
        self.params = dict(params)
        self.prefix = prefix
        self.ctx = ctx

    def tensor_specs(self, available: Set[str]) -> List[TensorSpec]:
        """The tensors this part reads; `available` holds the file's tensor names where naming has alternatives."""
        return []

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Takes the device tensors named by `tensor_specs` (roles already converted to their types)."""

    def name(self, suffix: str) -> str:
        return self.prefix + suffix

    def graph_key(self, step):
        """What, beyond the step's shape (rows, wanted places, block-table widths), fixes the launches this part makes
        for `step`: a hashable that the engine folds into the key under which it records and replays a decode step as
        a HIP graph.  A part whose launches follow a plan made per step (`step.shared`) returns the plan: a step with
        another plan is then another graph, and the graph keeps the plan alive.  None: nothing more."""
        return None


class Norm(Part):
    def forward(self, step, x: torch.Tensor, out: Optional[torch.Tensor], out32: Optional[torch.Tensor] = None,
                pick: Optional[torch.Tensor] = None) -> None:
        """out (activation type) and/or out32 (float32) = norm of the float32 rows x (of rows x[pick] when given)."""
        raise NotImplementedError

    def deferred(self, x: torch.Tensor):
        """The norm of x as a description that a product can carry out itself (ops.NormedRows), or None when this norm
        has no such form.  A block offers it to the part that follows; the part says whether it takes it."""
        return None


class PositionEncoding(Part):
    """Owns what a mixer needs to place a row at its position; for rotary forms a table of cos and sin, and which dims
    of a head rotate together."""

    #: "halves": dims i and i + R/2 are a pair; "interleaved": dims 2i and 2i + 1
    pairing = "halves"

    def rotation(self):
        """(cos_sin [positions, rotary_dim] float32 on the device, rotary_dim), cos of the pairs then sin; rotary_dim 0 rotates nothing."""
        raise NotImplementedError


@dataclass
class LayerCache:
    """What one run-order entry's mixer gets of the cache: its paged tensors by the names of its need, or per-request
    state."""
    group: int = -1                          # cache group of the pages (index for step.tables)
    tensors: Optional[Dict[str, torch.Tensor]] = None   # name -> [pages, *CacheTensor.page_shape(page_tokens)]
    writes: bool = True                      # False: this entry reads pages another entry wrote
    state: Optional[torch.Tensor] = None     # [slots, *StateNeed.shape]

    @property
    def k(self) -> torch.Tensor:
        """Keys of an attention cache: [pages, kv_heads, page_tokens, head_dim]."""
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:
        """Values of an attention cache: [pages, kv_heads, head_dim, page_tokens] (transposed within the page)."""
        return self.tensors["v"]


class Mixer(Part):
    #: True when forward wants the normed rows also as float32 (`h32`)
    wants_f32_input = False

    def takes_deferred_norm(self, step) -> bool:
        """Whether, for this step, forward accepts a Norm.deferred() description as h and h32 in place of tensors."""
        return False

    def cache_need(self) -> Union[PagedNeed, StateNeed, None]:
        return None

    def forward(self, step, h: torch.Tensor, out: torch.Tensor, accumulate: bool, cache: LayerCache,
                h32: Optional[torch.Tensor] = None) -> None:
        """out (float32 [T, hidden]) = or += mixer(h), h being the normed rows in the activation type."""
        raise NotImplementedError


class FeedForward(Part):
    wants_f32_input = False

    def takes_deferred_norm(self, step) -> bool:
        """As Mixer.takes_deferred_norm."""
        return False

    def forward(self, step, h: torch.Tensor, out: torch.Tensor, accumulate: bool, h32: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError


class Embedding(Part):
    def forward(self, step, out: torch.Tensor) -> None:
        """out (float32 [T, hidden]) = rows of the table for step.token_ids."""
        raise NotImplementedError

    def table(self) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    def forward(self, step, rows: torch.Tensor, logits: torch.Tensor) -> None:
        """logits (float32 [W, vocab]) for the normed rows (activation type [W, hidden])."""
        raise NotImplementedError


# ---------------------------------------------------------------------------
# registries: part name -> class
_REGISTRIES: Dict[str, Dict[str, Callable]] = {k: {} for k in ("norm", "position", "mixer", "feed_forward", "embedding", "head", "block")}


def register(family: str, kind: str, cls: Callable, replace: bool = False) -> None:
    table = _REGISTRIES[family]
    if kind in table and not replace and table[kind] is not cls:
        raise ValueError(f"a {family} part named {kind!r} is already registered")
    table[kind] = cls


def unregister(family: str, kind: str) -> None:
    _REGISTRIES[family].pop(kind, None)


def build_part(family: str, spec: PartSpec, ctx: BuildContext):
    table = _REGISTRIES[family]
    if spec.kind not in table:
        raise ValueError(f"no {family} part named {spec.kind!r} is registered (known: {sorted(table)})")
    part = table[spec.kind](spec.params, spec.prefix, ctx)
    part.kind = spec.kind
    return part
