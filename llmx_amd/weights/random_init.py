"""Seeded random weights, each tensor reproducible alone from (seed, its name).

A counter-based generator: element i of tensor `name` under `seed` is a function of (seed, name, i) only, so the host
(model folders for tests) and the device (in-place fill of models too large to stage) compute the same values up to the
rounding of log/cos.  Per-tensor streams keyed by name follow the reference's fixtures
(/root/reference/tests/fixture_minimax.py:42-83); the distributions are run options, not configuration.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..parts.spec import TensorSpec

_MASK = (1 << 64) - 1
GOLDEN = 0x9E3779B97F4A7C15


@dataclass(frozen=True)
class RandomInit:
    seed: int = 0
    std: float = 0.02            # matrices, tables, router matrices: N(0, std)
    norm_std: float = 0.0        # norm weights: 1 + N(0, norm_std)
    bias_range: float = 0.0      # bias vectors: U(-bias_range, bias_range)
    storage: str = "bfloat16"    # how matrices and tables are stored in a written folder ("bfloat16" | "float32")


def mix64(x: int) -> int:
    x &= _MASK
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _MASK
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _MASK
    x ^= x >> 31
    return x


def tensor_key(seed: int, name: str) -> int:
    h = 0xCBF29CE484222325  # FNV-1a over the name
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return mix64((seed * GOLDEN + h) & _MASK)


def distribution(spec: TensorSpec, init: RandomInit):
    """(kind, a, b): kind 0 = a + b * normal, kind 1 = uniform in [a, b).  What the spec states, else what its role says."""
    if spec.init is not None:
        kind = spec.init[0]
        if kind == "normal":
            return 0, float(spec.init[1]), float(spec.init[2])
        if kind == "uniform":
            return 1, float(spec.init[1]), float(spec.init[2])
        return 0, float(spec.init[1]), 0.0       # constant
    if spec.role == "norm":
        return 0, 1.0, init.norm_std
    if spec.role == "bias":
        return 1, -init.bias_range, init.bias_range
    if spec.role == "int":
        raise ValueError(f"no random rule for the integer table {spec.name}")
    return 0, 0.0, init.std


def _hash_elements(key: int, count: int, start: int = 0) -> np.ndarray:
    i = np.arange(start, start + count, dtype=np.uint64)
    x = np.uint64(key) + i * np.uint64(GOLDEN)
    x ^= x >> np.uint64(30)
    x *= np.uint64(0xBF58476D1CE4E5B9)
    x ^= x >> np.uint64(27)
    x *= np.uint64(0x94D049BB133111EB)
    x ^= x >> np.uint64(31)
    return x


def host_values(spec: TensorSpec, init: RandomInit) -> torch.Tensor:
    """The tensor's float32 values, computed on the host."""
    kind, a, b = distribution(spec, init)
    count = int(np.prod(spec.shape)) if spec.shape else 1
    out = np.empty(count, dtype=np.float32)
    key = tensor_key(init.seed, spec.name)
    chunk = 1 << 22
    with np.errstate(over="ignore"):
        for s in range(0, count, chunk):
            n = min(chunk, count - s)
            h = _hash_elements(key, n, s)
            hi = (h >> np.uint64(40)).astype(np.float32)
            if kind == 0:
                u1 = (hi + np.float32(1.0)) * np.float32(2.0 ** -24)
                u2 = ((h >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.float32) * np.float32(2.0 ** -24)
                z = np.sqrt(np.float32(-2.0) * np.log(u1, dtype=np.float32), dtype=np.float32) * np.cos(np.float32(6.2831853) * u2, dtype=np.float32)
                out[s:s + n] = np.float32(a) + np.float32(b) * z
            else:
                out[s:s + n] = np.float32(a) + np.float32(b - a) * (hi * np.float32(2.0 ** -24))
    return torch.from_numpy(out).view(spec.shape)


def stored_dtype(spec: TensorSpec, init: RandomInit) -> torch.dtype:
    """How a written folder stores the tensor: a stated type as it is, matrices and tables as the run asks."""
    if spec.dtype is not None:
        return getattr(torch, spec.dtype)
    if spec.role in ("matrix", "table"):
        return torch.bfloat16 if init.storage == "bfloat16" else torch.float32
    return torch.float32


def fill_random(t: torch.Tensor, spec: TensorSpec, init: RandomInit) -> None:
    """Fills the device tensor `t` in place with the values `host_values(spec, init)` computes, rounded to t's type
    (models too large to stage on the host)."""
    from .. import ops
    kind, a, b = distribution(spec, init)
    ops.fill_random(t, tensor_key(init.seed, spec.name), kind, a, b)
