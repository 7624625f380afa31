"""Perplexity of a sequence of token ids, in windows that each start from an empty history.

Follows the reference's definition (/root/reference/src/inference/perplexity.hpp:41-90): a window of `context` tokens
scores every token but its first (which is only context) with -(logit[target] - log sum exp(logits)) in double; a
rest shorter than two tokens is left out; windows run through the prompt path (portions of a step) or, with
`per_token`, one token a step through the decode path.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Sequence

import torch

MIN_WINDOW = 2


@dataclass
class PerplexityResult:
    context: int = 0
    used_tokens: int = 0
    scored_tokens: int = 0
    nll: float = 0.0
    windows: List[tuple] = field(default_factory=list)    # (scored tokens, their summed NLL) per window

    @property
    def mean_nll(self) -> float:
        return self.nll / self.scored_tokens

    @property
    def perplexity(self) -> float:
        return math.exp(self.mean_nll)


def rows_nll(logits: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
    """-(logit[target] - log sum exp) of each float32 row, in double."""
    z = logits.double()
    return torch.logsumexp(z, dim=1) - z.gather(1, targets.long().view(-1, 1)).view(-1)


def perplexity(engine, ids: Sequence[int], context: int = 0, max_chunks: int = 0, per_token: bool = False,
               portion: int = 512) -> PerplexityResult:
    ids = [int(t) for t in ids]
    if len(ids) < MIN_WINDOW:
        raise ValueError(f"perplexity: need at least {MIN_WINDOW} tokens")
    context = context or engine.max_positions
    if not MIN_WINDOW <= context <= engine.max_positions:
        raise ValueError(f"perplexity: context size must be between {MIN_WINDOW} and the engine's {engine.max_positions} positions")
    if max_chunks < 0:
        raise ValueError("perplexity: chunks must be nonnegative")
    result = PerplexityResult(context=context)
    begin = 0
    request = ("perplexity", id(result))
    while begin < len(ids):
        count = min(context, len(ids) - begin)
        if count < MIN_WINDOW or (max_chunks and len(result.windows) >= max_chunks):
            break
        window = ids[begin:begin + count]
        targets = torch.tensor(window[1:], dtype=torch.int64, device=engine.device)
        total = torch.zeros((), dtype=torch.float64, device=engine.device)
        engine.add_request(request)
        try:
            if per_token:
                for i in range(count - 1):          # the last token is a target only
                    row = engine.decode_one(request, window[i])
                    total += rows_nll(row.view(1, -1), targets[i:i + 1])[0]
            else:
                def take(first, out):
                    nonlocal total
                    n = min(out.shape[0], count - 1 - first)    # the window's last row predicts past it
                    if n > 0:
                        total += rows_nll(out[:n], targets[first:first + n]).sum()
                engine.score(request, window, portion, each=take)
        finally:
            engine.end_request(request)
        part = float(total)
        result.windows.append((count - 1, part))
        result.nll += part
        result.used_tokens += count
        result.scored_tokens += count - 1
        begin += count
    return result
