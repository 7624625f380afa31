"""Seeded random weights written in place on the device (models too large to stage on the host)."""

from __future__ import annotations

import torch

from ..parts.spec import TensorSpec
from .random_init import RandomInit, distribution, tensor_key


def fill_random(t: torch.Tensor, spec: TensorSpec, init: RandomInit) -> None:
    """Fills `t` with the values `random_init.host_values(spec, init)` computes, rounded to t's type."""
    from .. import ops
    kind, a, b = distribution(spec, init)
    ops.fill_random(t, tensor_key(init.seed, spec.name), kind, a, b)
