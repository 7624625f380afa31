"""Token embedding and the language-model head.

x[t] = table[id[t]] widened to float32 (/root/reference/src/model/arch/blocks.hpp:95-97); logits = rows . W^T in
float32 for the wanted rows only (:267-272).  A tied head reads the embedding's table.
"""

from __future__ import annotations

import torch

from .. import ops
from .base import Embedding, Head, register
from .spec import TensorSpec


class TokenEmbedding(Embedding):
    """params: vocab, hidden; tensor <prefix>weight (vocab, hidden)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.weight = None

    def tensor_specs(self, available):
        return [TensorSpec(self.name("weight"), (self.vocab, self.hidden), "table")]

    def load(self, tensors):
        self.weight = tensors[self.name("weight")]

    def table(self):
        return self.weight

    def forward(self, step, out):
        ops.embed_gather(self.weight, step.token_ids, out)


class LinearHead(Head):
    """params: vocab, hidden, tied (bool); tensor <prefix>weight (vocab, hidden) unless tied."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.tied = bool(params.get("tied", False))
        self.weight = None

    def tensor_specs(self, available):
        return [] if self.tied else [TensorSpec(self.name("weight"), (self.vocab, self.hidden), "table")]

    def load(self, tensors):
        if not self.tied:
            self.weight = tensors[self.name("weight")]

    def tie(self, table: torch.Tensor) -> None:
        self.weight = table

    def forward(self, step, rows, logits):
        ops.gemm(rows, self.weight, logits)


register("embedding", "token_embedding", TokenEmbedding)
register("head", "linear", LinearHead)
