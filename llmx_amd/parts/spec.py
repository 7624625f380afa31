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
    """
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    into: Optional[Tuple[str, Tuple[int, ...], tuple]] = None

    ROLES = ("matrix", "table", "norm", "bias", "router", "int")


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
class KVNeed:
    """A mixer that keeps keys and values of every position (window None) or of the last `window` positions."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


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
