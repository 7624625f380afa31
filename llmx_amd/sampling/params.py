"""Sampling settings, their defaults and ranges, and the generator each request owns.

Names, defaults and ranges are the reference's (/root/reference/src/inference/sampler.hpp:43-65); the generator is its
xorshift64 (:21-32).
"""

from __future__ import annotations

from dataclasses import dataclass

MAX_EXACT_TOP_K = 1024       # kept sets up to this size are ranked whole in LDS; larger ones are searched by histograms
_M64 = (1 << 64) - 1


@dataclass
class SamplingParams:
    max_tokens: int = 64             # tokens generated at most
    temp: float = 0.8                # 0 is greedy
    top_k: int = 40                  # 0 keeps every token
    top_p: float = 0.95              # 1 keeps every token
    min_p: float = 0.0               # drops tokens below this share of the likeliest token's weight
    penalty: float = 1.0             # repetition penalty, 1 is none
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    seed: int = 0                    # 0 keeps the generator's fixed default state
    ignore_eos: bool = False         # the end token is never drawn
    stop: tuple = ()                 # sequences of token ids; generation ends when the generated ids end with one

    def validate(self) -> "SamplingParams":
        def bad(name, why):
            return ValueError(f"sampling: {name} {why}")
        if self.max_tokens < 1:
            raise bad("max_tokens", "must be at least 1")
        if not self.temp >= 0.0:
            raise bad("temp", "must be at least 0")
        if self.top_k < 0:
            raise bad("top_k", "must be at least 0")
        if not 0.0 <= self.top_p <= 1.0:
            raise bad("top_p", "must lie in [0, 1]")
        if not 0.0 <= self.min_p <= 1.0:
            raise bad("min_p", "must lie in [0, 1]")
        if not self.penalty >= 1.0:
            raise bad("penalty", "must be at least 1")
        if not -2.0 <= self.presence_penalty <= 2.0:
            raise bad("presence_penalty", "must lie in [-2, 2]")
        if not -2.0 <= self.frequency_penalty <= 2.0:
            raise bad("frequency_penalty", "must lie in [-2, 2]")
        if self.seed < 0 or self.seed > _M64:
            raise bad("seed", "must fit 64 unsigned bits")
        self.stop = normalize_stop(self.stop)
        return self

    @property
    def greedy(self) -> bool:
        return self.temp <= 0.0

    @property
    def penalized(self) -> bool:
        return (self.penalty > 0.0 and self.penalty != 1.0) or self.presence_penalty != 0.0 or self.frequency_penalty != 0.0


MAX_STOPS, MAX_STOP_TOKENS = 16, 256


def normalize_stop(stop) -> tuple:
    """A tuple of tuples of token ids from one sequence of ids or several.

    The reference stops on a text (/root/reference/src/inference/generate.hpp:33, at most 16 of 256 bytes each on its
    server); without a tokenizer a sequence of token ids stands for the text.
    """
    if not stop:
        return ()
    seqs = [stop] if all(isinstance(t, int) for t in stop) else list(stop)
    out = []
    for s in seqs:
        s = tuple(int(t) for t in s)
        if not s or len(s) > MAX_STOP_TOKENS or any(t < 0 for t in s):
            raise ValueError(f"sampling: a stop sequence holds 1 to {MAX_STOP_TOKENS} token ids")
        out.append(s)
    if len(out) > MAX_STOPS:
        raise ValueError(f"sampling: stop holds at most {MAX_STOPS} sequences")
    return tuple(out)


class XorShift64:
    """x ^= x << 13; x ^= x >> 7; x ^= x << 17; unit = (next >> 40) / 2^24 as a float."""

    def __init__(self, seed: int = 0):
        self.state = 0x9E3779B97F4A7C15
        if seed:
            self.state = seed & _M64

    def next(self) -> int:
        x = self.state
        x ^= (x << 13) & _M64
        x ^= x >> 7
        x ^= (x << 17) & _M64
        self.state = x
        return x

    def unit(self) -> float:
        return (self.next() >> 40) * (1.0 / 16777216.0)
