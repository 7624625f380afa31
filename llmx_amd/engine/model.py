"""A model built from a ModelSpec: its parts, the tensors they read, and what each cache number needs."""

from __future__ import annotations

from typing import Dict, List, Set, Union

import torch

from ..parts import base as parts_base
from ..parts.base import BuildContext, build_part
from ..parts.spec import ModelSpec, PagedNeed, StateNeed, TensorSpec


def build_block(spec, ctx: BuildContext):
    table = parts_base._REGISTRIES["block"]
    if spec.arrangement not in table:
        raise ValueError(f"no block arrangement named {spec.arrangement!r} is registered (known: {sorted(table)})")
    return table[spec.arrangement](spec, ctx)


class BuiltModel:
    def __init__(self, spec: ModelSpec, ctx: BuildContext):
        spec.check()
        self.spec = spec
        self.ctx = ctx
        self.embedding = build_part("embedding", spec.embedding, ctx)
        self.blocks = [build_block(b, ctx) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, ctx)
        self.head = build_part("head", spec.head, ctx)

    def parts(self):
        out = [self.embedding]
        for b in self.blocks:
            out.extend(b.parts())
        out += [self.final_norm, self.head]
        return out

    def tensor_specs(self, available: Set[str] = frozenset()) -> List[TensorSpec]:
        specs: List[TensorSpec] = []
        for p in self.parts():
            specs.extend(p.tensor_specs(available))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self.parts():
            p.load(tensors)
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.table())

    def cache_needs(self) -> List[Union[PagedNeed, StateNeed, None]]:
        """For each cache number of the run order, what its writer keeps."""
        needs: Dict[int, Union[PagedNeed, StateNeed, None]] = {}
        for e in self.spec.run_order:
            need = self.blocks[e.layer].mixer.cache_need()
            if e.writes:
                needs[e.cache] = need
            elif needs[e.cache] != need:
                raise ValueError(f"layer {e.layer} reads cache {e.cache}, which holds {needs[e.cache]}, but needs {need}")
        return [needs[i] for i in range(len(needs))]
