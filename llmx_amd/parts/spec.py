"""Declarative description of a model: which parts make each layer and in which order layers run.

An architecture turns its typed configuration into a `ModelSpec`; nothing below
that (builder, weights loader, cache manager, step function, scheduler) knows
which architecture it came from.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part reads from the file, by its full name.

    role: "matrix" / "table" keep bfloat16 (or the stored 32 bits) in the bf16 path and are widened to float32 in the
          32-bit path; "norm" and "bias" vectors and "router" matrices are always float32; "int" tables are int32.
    into: (target name, target shape, index): the tensor is one slice of a larger device tensor that the part reads
          instead; the loader allocates the target once and copies each file tensor from the host straight into
          target[index], so the slices are never on the device beside their fused copy.
    dtype: the tensor's type on the device ("float32" | "bfloat16" | "int32"), whatever the file stores and whichever
          path runs; None: what the role says.  A part whose parameter is of a kind the roles do not know (a decay
          kept in float32, a table of 32-bit ids) states it here; loader and random weights follow it.
    init: how random weights fill it: ("normal", mean, std) | ("uniform", low, high) | ("constant", value); None: what
          the role says (matrices N(0, std), norm weights 1 + N(0, norm_std), biases U(-range, range) of the run's
          RandomInit).
    """
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    into: Optional[Tuple[str, Tuple[int, ...], tuple]] = None
    dtype: Optional[str] = None
    init: Optional[Tuple] = None

    ROLES = ("matrix", "table", "norm", "bias", "router", "int")
    DTYPES = ("float32", "bfloat16", "int32")
    INITS = ("normal", "uniform", "constant")

    def __post_init__(self):
        if self.role not in self.ROLES:
            raise ValueError(f"tensor {self.name}: role {self.role!r} is not one of {self.ROLES}")
        if self.dtype is not None and self.dtype not in self.DTYPES:
            raise ValueError(f"tensor {self.name}: dtype {self.dtype!r} is not one of {self.DTYPES}")
        if self.init is not None:
            kind = self.init[0] if self.init else None
            if kind not in self.INITS or len(self.init) != (2 if kind == "constant" else 3):
                raise ValueError(f"tensor {self.name}: init {self.init!r} is not (\"normal\", mean, std), (\"uniform\", low, high) or (\"constant\", value)")


@dataclass
class PartSpec:
    """A part by the name it is registered under, its parameters, and the prefix of its tensors' names."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    prefix: str = ""


@dataclass
class BlockSpec:
    """One layer: its parts and the name of their arrangement ("prenorm": x += mixer(norm(x)); x += ffn(norm(x))).

    The four named parts are what most arrangements have; an arrangement that needs more (norms after the mixer and
    the feed-forward, a second feed-forward, a gate) finds them in `extra` by the names it gives them, each with the
    family ("norm", "mixer", "feed_forward", ...) it is built from.  The arrangement class builds what it uses and
    lists it in `parts()`; the engine asks a block's `mixer` for what its cache number holds.
    """
    mixer_norm: PartSpec
    mixer: PartSpec
    ffn_norm: PartSpec
    ffn: PartSpec
    arrangement: str = "prenorm"
    extra: Dict[str, Tuple[str, PartSpec]] = field(default_factory=dict)   # name -> (family, part)


@dataclass(frozen=True)
class RunEntry:
    """One item of the run order: run block `layer` with cache `cache`.

    A layer may be named by several entries (its weights run twice); two entries may name one cache, the later ones
    with writes=False reading what the first wrote.
    """
    layer: int
    cache: int
    writes: bool = True


@dataclass(frozen=True)
class CacheTensor:
    """One tensor a mixer keeps for every token of a request, in pages.

    shape:      the values of one token, e.g. (kv_heads, head_dim) for keys, (latent_width,) for one latent a token;
    dtype:      a torch dtype name, or None for the engine's activation type;
    token_axis: where a page's token axis sits among `shape`'s axes: a page of this tensor has `shape` with
                `page_tokens` put in at that place.  (kv_heads, head_dim) with token_axis 1 gives pages
                [kv_heads, page_tokens, head_dim] (keys: a token's dims lie together); token_axis 2 gives
                [kv_heads, head_dim, page_tokens] (values stored transposed within the page).
    """
    name: str
    shape: Tuple[int, ...]
    dtype: Optional[str] = None
    token_axis: int = 0

    def page_shape(self, page_tokens: int) -> Tuple[int, ...]:
        if not 0 <= self.token_axis <= len(self.shape):
            raise ValueError(f"cache tensor {self.name}: token_axis {self.token_axis} outside its {len(self.shape)} axes")
        return tuple(self.shape[:self.token_axis]) + (int(page_tokens),) + tuple(self.shape[self.token_axis:])


@dataclass(frozen=True)
class PagedNeed:
    """A mixer that keeps tensors of every position (window None) or of the last `window` positions, in pages.  The
    engine allocates what is listed (one arena a tensor and cache group) and knows nothing else of it; mixers with equal
    needs share a cache group: one page pool and one block table a request."""
    tensors: Tuple[CacheTensor, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged cache need lists at least one tensor and no name twice, not {names}")


def KVNeed(kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedNeed:
    """The need of softmax attention: keys [kv_heads, token, head_dim] and values [kv_heads, head_dim, token] (transposed
    within the page) in the activation type."""
    return PagedNeed((CacheTensor("k", (int(kv_heads), int(head_dim)), None, 1), CacheTensor("v", (int(kv_heads), int(head_dim)), None, 2)), window)


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a fixed-size state per request: `shape` values of `dtype` (a torch dtype name)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    blocks: List[BlockSpec]
    run_order: List[RunEntry]
    final_norm: PartSpec
    head: PartSpec
    eos_token_id: Optional[int] = None
    bos_token_id: Optional[int] = None

    def check(self) -> None:
        n_caches = 0
        writers = set()
        for e in self.run_order:
            if not 0 <= e.layer < len(self.blocks):
                raise ValueError(f"run order names layer {e.layer}, outside the model's {len(self.blocks)} layers")
            if e.writes:
                if e.cache in writers:
                    raise ValueError(f"run order lets two entries write cache {e.cache}")
                writers.add(e.cache)
            elif e.cache not in writers:
                raise ValueError(f"run order reads cache {e.cache} before any entry writes it")
            n_caches = max(n_caches, e.cache + 1)
        if writers != set(range(n_caches)):
            raise ValueError("run order leaves a cache number without a writer")
