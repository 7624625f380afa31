"""Configurations drawn at random through the engine, against the plain implementation.

The two tiny configurations fix two points of the space of sizes; this file walks through more of it: head widths in
steps of 16 up to 256, head counts and groups that are no power of two (one KV head, one query head a group, five
groups), rotation of none, part or all of a head, one expert, an odd number of experts, every pick count, widths
that are only multiples of two, odd vocabularies, all page sizes.  Each configuration runs whole, with the last 32
tokens one by one, in portions of changing size, and as six requests mixed through a pool for four, in both dtypes; the cuttings must agree bit for bit and the
whole run must agree with the plain implementation within the bounds of test_engine_gpu (the plain implementation
is given the engine's expert picks, each checked to be one of the best within rounding).  A size that a kernel does
not take must be refused with an error, never computed wrongly: a refusal would fail here by name.
"""

from __future__ import annotations

import random

import pytest
import torch

import helpers
import test_engine_gpu as engine_tests
from llmx_amd import MiniMaxM3Config, RandomInit

pytestmark = pytest.mark.gpu


def drawn(seed: int, wide: bool):
    rng = random.Random(7000 + seed)
    head_dim = rng.choice(range(16, 257, 16))
    kv_heads = rng.choice([1, 2, 3, 4, 5])
    heads = kv_heads * rng.choice([1, 2, 3, 4, 6, 8])
    rotary = rng.choice([0, 2 * rng.randrange(1, head_dim // 2 + 1), head_dim])
    experts = rng.choice([1, 3, 8, 12, 17, 40])
    cfg = dict(vocab_size=rng.choice([8191, 20001, 33000] if wide else [97, 256, 331, 1000, 4099]),
               hidden_size=2 * (rng.randrange(200, 700) if wide else rng.randrange(12, 160)),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
               rotary_dim=rotary, rope_theta=rng.choice([1e4, 5e5, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-5]),
               num_local_experts=experts, num_experts_per_tok=rng.randrange(1, min(experts, 6) + 1),
               intermediate_size=2 * (rng.randrange(100, 500) if wide else rng.randrange(8, 120)),
               routed_scaling_factor=rng.choice([1.0, 2.5, 0.7]), norm_topk_prob=rng.choice([True, False]),
               tie_word_embeddings=False, max_position_embeddings=2048)
    init = RandomInit(seed=rng.randrange(100), std=rng.choice([0.02, 0.05]), norm_std=rng.choice([0.0, 0.1]),
                      bias_range=rng.choice([0.0, 0.1]), storage="bfloat16")
    return cfg, init, rng.choice([4, 8, 16, 32, 64])


CASES = [(seed, False, 75) for seed in range(16)] + [(seed, True, 300) for seed in range(200, 204)]


def test_the_draws_cover_the_options():
    """Guards the generator itself: the cases below do reach the corners they are meant to."""
    cfgs = [drawn(seed, wide)[0] for seed, wide, _ in CASES]
    for cfg in cfgs:
        MiniMaxM3Config(**cfg)
    assert {c["rotary_dim"] == 0 for c in cfgs} == {True, False}
    assert any(0 < c["rotary_dim"] < c["head_dim"] for c in cfgs) and any(c["rotary_dim"] == c["head_dim"] for c in cfgs)
    assert any(c["num_local_experts"] == 1 for c in cfgs) and any(c["num_local_experts"] % 2 for c in cfgs)
    assert any(c["num_key_value_heads"] == c["num_attention_heads"] for c in cfgs) and any(c["num_key_value_heads"] == 1 for c in cfgs)
    assert any(c["head_dim"] > 128 for c in cfgs) and any(c["head_dim"] % 32 for c in cfgs)
    assert any(c["hidden_size"] % 8 for c in cfgs) and any(c["intermediate_size"] % 8 for c in cfgs)
    assert {drawn(seed, wide)[2] for seed, wide, _ in CASES} == {4, 8, 16, 32, 64}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed,wide,length", CASES, ids=lambda v: str(v))
def test_a_drawn_configuration(seed, wide, length, dtype):
    name = f"drawn{seed}"
    helpers.TINY[name] = drawn(seed, wide)
    engine = engine_tests.make_engine(name, dtype)
    engine.observer = helpers.RoutingRecorder(helpers.TINY[name][0]["num_hidden_layers"])
    tokens = helpers.tokens_for(name, length, 0)
    whole = engine_tests.run_whole(engine, "w", tokens)
    assert torch.isfinite(whole).all()
    # Among hundreds of rows drawn without care some router keys lie closer than float32 resolves (1e-7 apart), so in
    # both dtypes the plain implementation takes the engine's picks, after checking each against the engine's own router
    # logits, and those logits against the plain ones.
    rounded = dtype == "bfloat16"
    want = helpers.plain_logits_with_picks(name, tokens, engine.observer.of("w", length), rounded=rounded,
                                           engine_logits=engine.observer.logits_of("w", length))
    tol = engine_tests.BF16_TOL if rounded else engine_tests.F32_TOL
    err, scale = float((whole.double() - want).abs().max()), float(want.abs().max())
    assert err <= tol * scale, f"{helpers.TINY[name][0]} {dtype}: max error {err:.3e} against scale {scale:.3e}"
    one_by_one = engine_tests.run_cut(engine, "d", tokens, [(0, length - 32)] + [(i, i + 1) for i in range(length - 32, length)])
    assert torch.equal(one_by_one, whole), f"{helpers.TINY[name][0]}: decoding one by one differs from the whole prompt"
    cut = engine_tests.run_cut(engine, "p", tokens, helpers.portions(length))
    assert torch.equal(cut, whole), f"{helpers.TINY[name][0]}: portions differ from the whole prompt"
    assert engine.cache.pages_in_use() == 0
    # six requests through a pool for four, mixed in steps: each must have the bits of its run alone
    _, prompts, mixed = engine_tests.run_mixed(name, dtype)
    for i, prompt in enumerate(prompts):
        assert torch.equal(mixed[i], engine_tests.run_whole(engine, "w", prompt)), \
            f"{helpers.TINY[name][0]}: request {i} in the mix differs from its run alone"
