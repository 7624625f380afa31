"""The arrangement of a layer's parts.

"prenorm": x += mixer(norm(x)); x += ffn(norm(x)) with the residual x in float32: the arrangement of
/root/reference/src/model/arch/minimax_m3.hpp:247-287 (norm, mixer joined into the residual, norm, feed-forward joined).
"""

from __future__ import annotations

import torch

from .base import BuildContext, LayerCache, build_part, register
from .spec import BlockSpec


class PreNormBlock:
    graph_safe = True   # see Part.graph_safe

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx)
        self.mixer = build_part("mixer", spec.mixer, ctx)
        self.ffn_norm = build_part("norm", spec.ffn_norm, ctx)
        self.ffn = build_part("feed_forward", spec.ffn, ctx)

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        T, E = x.shape
        h = step.buf("block.h", (T, E), step.act_dtype)
        h32 = step.buf("block.h32", (T, E), torch.float32) if self.mixer.wants_f32_input else None
        self.mixer_norm.forward(step, x, h, h32)
        self.mixer.forward(step, h, x, True, cache, h32)
        h32 = step.buf("block.h32", (T, E), torch.float32) if self.ffn.wants_f32_input else None
        self.ffn_norm.forward(step, x, h, h32)
        self.ffn.forward(step, h, x, True, h32)


register("block", "prenorm", PreNormBlock)
