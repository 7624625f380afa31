"""RMSNorm: y = x * (r * w), r = 1/sqrt(mean(x^2) + eps), all in float32.

Order of operations as the reference computes it (/root/reference/src/backends/cpu/cpu_backend.hpp:1437-1459): the
reciprocal root times the weight is formed first, then multiplied into x.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from .base import Norm, register
from .spec import TensorSpec


class RMSNorm(Norm):
    """params: width, eps; tensor: <prefix>weight (width,)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self, available):
        return [TensorSpec(self.name("weight"), (self.width,), "norm")]

    def load(self, tensors):
        self.weight = tensors[self.name("weight")]

    def forward(self, step, x, out, out32=None, pick=None):
        ops.rmsnorm(x, self.weight, self.eps, out, out32, pick)

    def deferred(self, x):
        return ops.NormedRows(x, self.weight, self.eps)


register("norm", "rmsnorm", RMSNorm)
