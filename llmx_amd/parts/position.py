"""Position encodings.

Rotary tables follow the reference's float32 arithmetic (/root/reference/src/model/rope.hpp:25-28,203-210):
freq_i = 1.0f / powf(theta, 2.0f*i/R), angle = (float)pos * freq_i, cos and sin of that angle, one table for all
layers, pairs (i, i + R/2) of each head rotated (NeoX halves).
"""

from __future__ import annotations

import numpy as np
import torch

from .base import PositionEncoding, register

PAIRINGS = ("halves", "interleaved")


def neox_table(positions: int, rotary_dim: int, theta: float) -> np.ndarray:
    """[positions, rotary_dim] float32: cos of the rotary_dim/2 pairs, then sin.

    Every value is what correctly rounded float32 functions give: the power, the cosine and the sine are computed in
    float64 from their float32 arguments and rounded once (vectorised float32 routines lose bits in the range reduction
    of large angles, and a position of 65,536 is a large angle); products and the division are float32.
    """
    half = rotary_dim // 2
    if half == 0:
        return np.zeros((positions, 0), dtype=np.float32)
    i = np.arange(half, dtype=np.float32)
    exponent = (np.float32(2.0) * i / np.float32(rotary_dim)).astype(np.float32)
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    freq = (np.float32(1.0) / power).astype(np.float32)
    pos = np.arange(positions, dtype=np.float32)[:, None]
    angle = (pos * freq[None, :]).astype(np.float32).astype(np.float64)
    return np.concatenate([np.cos(angle), np.sin(angle)], axis=1).astype(np.float32)


class PartialRotary(PositionEncoding):
    """params: rotary_dim (even, at most head_dim; 0 rotates nothing), theta, head_dim, pairing ("halves", the default:
    dims i and i + rotary_dim/2 rotate together; "interleaved": dims 2i and 2i + 1)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.pairing = str(params.get("pairing", "halves"))
        if self.pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {self.pairing!r} is not one of {sorted(PAIRINGS)}")
        self.rotary_dim = int(params["rotary_dim"])
        self.theta = float(params["theta"])
        head_dim = int(params["head_dim"])
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= head_dim:
            raise ValueError(f"rotary width {self.rotary_dim} must be even and at most the head width {head_dim}")
        table = neox_table(ctx.max_positions, self.rotary_dim, self.theta)
        self.cos_sin = torch.from_numpy(table).to(ctx.device)

    def rotation(self):
        return self.cos_sin, self.rotary_dim


class NoPosition(PositionEncoding):
    """Leaves rows as they are."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.cos_sin = torch.zeros((max(1, ctx.max_positions), 0), dtype=torch.float32, device=ctx.device)

    def rotation(self):
        return self.cos_sin, 0


register("position", "rotary_neox_partial", PartialRotary)
register("position", "none", NoPosition)
