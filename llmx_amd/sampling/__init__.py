"""Sampling: settings, per-request generators, and the device sampler."""

from .params import MAX_EXACT_TOP_K, SamplingParams, XorShift64

__all__ = ["MAX_EXACT_TOP_K", "SamplingParams", "XorShift64", "Sampler"]


def __getattr__(name):
    if name == "Sampler":
        from .sampler import Sampler
        return Sampler
    raise AttributeError(name)
