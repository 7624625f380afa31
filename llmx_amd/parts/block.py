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

    @staticmethod
    def normed(step, norm, part, x):
        """(h, h32) for `part`: the norm's description where the norm has one and the part carries it out in its own
        products for this step (a step of very few rows, where a norm kernel of its own costs more than its work);
        otherwise the norm runs here."""
        later = norm.deferred(x)
        if later is not None and part.takes_deferred_norm(step):
            return later, later
        T, E = x.shape
        h = step.buf("block.h", (T, E), step.act_dtype)
        h32 = step.buf("block.h32", (T, E), torch.float32) if part.wants_f32_input else None
        norm.forward(step, x, h, h32)
        return h, h32

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        h, h32 = self.normed(step, self.mixer_norm, self.mixer, x)
        self.mixer.forward(step, h, x, True, cache, h32)
        h, h32 = self.normed(step, self.ffn_norm, self.ffn, x)
        self.ffn.forward(step, h, x, True, h32)


register("block", "prenorm", PreNormBlock)
