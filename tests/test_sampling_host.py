"""Sampling settings and the per-request generator (the device kernels are tested on the GPU)."""

import pytest

import sampler_reference
from llmx_amd.sampling import SamplingParams, XorShift64


def test_generator_follows_the_xorshift_definition():
    """First outputs recomputed from the definition (/root/reference/src/inference/sampler.hpp:21-32)."""
    def step(x):
        m = (1 << 64) - 1
        x ^= (x << 13) & m
        x ^= x >> 7
        x ^= (x << 17) & m
        return x
    g, x = XorShift64(), 0x9E3779B97F4A7C15
    for _ in range(5):
        x = step(x)
        assert g.next() == x
    assert XorShift64(0).state == 0x9E3779B97F4A7C15       # seed 0 keeps the default state
    g = XorShift64(12345)
    x = step(12345)
    assert g.unit() == (x >> 40) / 16777216.0 and 0.0 <= g.unit() < 1.0
    a, b = XorShift64(7), XorShift64(7)
    assert [a.unit() for _ in range(10)] == [b.unit() for _ in range(10)]


def test_defaults_and_ranges():
    d = SamplingParams()
    assert (d.max_tokens, d.temp, d.top_k, d.top_p, d.min_p, d.penalty, d.presence_penalty, d.frequency_penalty, d.seed, d.ignore_eos) == \
        (64, 0.8, 40, 0.95, 0.0, 1.0, 0.0, 0.0, 0, False)
    d.validate()
    for bad in (dict(max_tokens=0), dict(temp=-0.1), dict(top_k=-1), dict(top_p=1.5), dict(min_p=-0.1), dict(penalty=0.5),
                dict(presence_penalty=3.0), dict(frequency_penalty=-2.5), dict(seed=-1)):
        with pytest.raises(ValueError, match="sampling: " + next(iter(bad))):
            SamplingParams(**bad).validate()
    # a nucleus over the whole row and a top-k of any size are taken, as in the reference (sampler.hpp:149-252)
    SamplingParams(top_k=0, top_p=0.9).validate()
    SamplingParams(top_k=5000, top_p=1.0).validate()
    SamplingParams(temp=0.0, top_k=0, top_p=0.5).validate()     # greedy reads neither
    assert SamplingParams(temp=0.0).greedy and not SamplingParams().greedy and SamplingParams(penalty=1.2).penalized


def test_reference_transcription_on_small_rows():
    """The slow sampler the GPU tests compare with: greedy vectors of /root/reference/tests/sampler.cpp:95-98 and simple draws."""
    s = sampler_reference.sample
    assert s([0.5, 2.0, -1.0, 1.5], 0.0, 0, 1.0, 0.0, 0.3) == 1
    assert s([1.0, 3.0, 0.0, 3.0], 0.0, 0, 1.0, 0.0, 0.3) == 1
    assert s([3.0, 3.0, 3.0], 0.0, 0, 1.0, 0.0, 0.9) == 0
    row = [0.0, 0.0, 0.0, 0.0]
    assert [s(row, 1.0, 0, 1.0, 0.0, r) for r in (0.0, 0.3, 0.6, 0.9)] == [0, 1, 2, 3]       # equal weights: the draw walks ids in order
    assert s([0.2, 1.5, -0.3, 1.1], 1.0, 1, 1.0, 0.0, 0.99) == 1                               # top_k 1 keeps the best only
    assert s([0.0, 5.0, 4.9, -3.0], 1.0, 3, 0.5, 0.0, 0.99) == 1                               # the nucleus is the best alone
    assert s([0.0, 5.0, 4.9, -3.0], 1.0, 3, 0.9, 0.0, 0.99) == 2                               # two in the nucleus, drawn best first
    assert s([0.0, 1.0, 0.5, 0.9], 1.0, 0, 1.0, 0.95, 0.99) == 1                               # min_p drops all but the best
    assert s([2.0, 1.0, 5.0], 1.0, 0, 1.0, 0.0, 0.5, skip=2) in (0, 1)                         # the masked id is never drawn
