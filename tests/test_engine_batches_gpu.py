"""Decode steps of many requests, and a long portion beside decoding requests: the compositions a serving loop issues.

Seventeen, thirty-three and sixty-four requests of different lengths are decoded together for 40 steps with graph
replays on; some of them pass a block table's width of 64 pages on the way and some the 896 tokens where the split
contexts' partial results get more slots.  Every request's rows must be the bits of its run alone (the reference's
"two sequences batched == each alone", /root/reference/tests/kv_cache.cpp, docs/TESTS.md:863-866).  Such steps take
kernels that steps of a few requests do not: the weight-streaming product with two and four tiles of rows and with two
strips, routed products through the tiled kernels from 17 token rows on, routing and grouping as two launches, more
attention items than one plan splits.  The launch witness (ops.take_launches) says which forms ran, so that a dispatch
that silently fell to the universal kernels fails here and not only in a benchmark.
"""

from __future__ import annotations

import random

import pytest
import torch

import helpers
from helpers import INIT_A, INIT_B, TINY_A, TINY_B, model_folder

pytestmark = pytest.mark.gpu

DECODE_STEPS = 40

# configuration A with room for contexts beyond 64 pages of 16 tokens
helpers.TINY.setdefault("A16L", (dict(TINY_A, max_position_embeddings=2048), INIT_A, 16))
helpers.TINY.setdefault("A4L", (dict(TINY_A, max_position_embeddings=2048), INIT_A, 4))

UNIVERSAL = {"gemm_generic", "gemm_generic.grouped", "attention.generic"}
MATRIX_CORE_BF16 = {"gemm_skinny", "gemm_skinny.two_strips", "gemm_skinny.normed", "gemm_skinny.grouped", "gemm_skinny.grouped_normed",
                    "gemm_tile.64", "gemm_tile.wide", "gemm_tile.bounded", "gemm_tile.grouped_64", "gemm_tile.grouped_128",
                    "gemm_tile.grouped_wide", "gemm_tile.grouped_bounded", "attention.tiles128", "attention.tiles", "attention.direct",
                    "attention.partial", "attention.split4", "attention.merge"}


def lengths_for(n_requests: int, page: int, seed: int):
    """Prompt lengths: most short and all different in their last page, a few that pass 64 pages while they are decoded,
    a few that pass 896 tokens."""
    rng = random.Random(seed)
    lengths = [rng.randrange(1, 150) for _ in range(n_requests)]
    edge = 64 * page
    for j, at in enumerate((edge - 3, edge - 20, edge - DECODE_STEPS + 1)):
        lengths[(5 * j + 1) % n_requests] = at
    for j, at in enumerate((896 - 2, 896 - 25)):
        lengths[(7 * j + 3) % n_requests] = at
    return lengths


def decode_together(engine, prompts, tails):
    """Prefills every prompt (a few requests a step), then feeds tails[i][s] of every request in step s.  Returns, for
    each request, the logits [DECODE_STEPS, vocab] of its decoded tokens."""
    from llmx_amd.engine import StepEntry
    n = len(prompts)
    for i in range(n):
        engine.add_request(i)
    for a in range(0, n, 5):
        engine.step([StepEntry(i, prompts[i], []) for i in range(a, min(n, a + 5))])
    rows = [[] for _ in range(n)]
    for s in range(DECODE_STEPS):
        out = engine.step([StepEntry(i, [tails[i][s]], [0]) for i in range(n)]).clone()
        for i in range(n):
            rows[i].append(out[i])
    for i in range(n):
        engine.end_request(i)
    return [torch.stack(r) for r in rows]


def alone(engine, prompt, tail):
    """The same request by itself: one step over prompt and tail, the logits of the tail's places."""
    from llmx_amd.engine import StepEntry
    engine.add_request("alone")
    L = len(prompt)
    out = engine.step([StepEntry("alone", prompt + tail, list(range(L, L + len(tail))))]).clone()
    engine.end_request("alone")
    return out


def check_decoding_together(engine, vocab, n_requests, page, seed):
    from llmx_amd import ops
    rng = random.Random(100 + seed)
    lengths = lengths_for(n_requests, page, seed)
    prompts = [[rng.randrange(vocab) for _ in range(n)] for n in lengths]
    tails = [[rng.randrange(vocab) for _ in range(DECODE_STEPS)] for _ in lengths]
    replays_before = engine.graph_replays
    ops.take_launches()
    together = decode_together(engine, prompts, tails)
    launched = ops.take_launches()
    assert engine.cache.pages_in_use() == 0
    assert engine.graph_replays - replays_before >= DECODE_STEPS // 2, "decode steps of this many requests were not replayed as graphs"
    for i in range(n_requests):
        want = alone(engine, prompts[i], tails[i])
        assert torch.equal(together[i], want), (f"request {i} of {n_requests} (prompt of {lengths[i]} tokens) decoded beside the others "
                                                f"differs from its run alone")
    return launched


@pytest.mark.parametrize("n_requests", [17, 33, 64])
@pytest.mark.parametrize("name,dtype", [("A16L", "bfloat16"), ("A4L", "float32"), ("B", "bfloat16"), ("B", "float32")])
def test_many_requests_decoded_together_equal_each_alone(name, dtype, n_requests):
    from llmx_amd.engine import Engine
    cfg, _, page = helpers.TINY[name]
    engine = Engine.load(model_folder(name), dtype=dtype, kv_tokens=16384, page_tokens=page, max_requests=n_requests + 1)
    assert engine.graphs
    launched = check_decoding_together(engine, cfg["vocab_size"], n_requests, page, seed=n_requests)
    if dtype == "float32":
        # the true 32-bit path: no kernel that rounds to bfloat16 anywhere
        assert not set(launched) & MATRIX_CORE_BF16, f"a float32 engine launched {sorted(set(launched) & MATRIX_CORE_BF16)}"
        assert {"gemm_generic", "gemm_generic.grouped", "attention.generic"} <= set(launched)
        assert any(k.startswith("gemm_f32") for k in launched), "the router's product did not run on the float32 matrix instruction"
    elif name == "A16L":
        # head size 16 on pages of 16, K a multiple of 64: everything runs on the matrix cores
        assert not set(launched) & UNIVERSAL, f"the bfloat16 engine fell to {sorted(set(launched) & UNIVERSAL)}"
        assert "gemm_skinny" in launched and "gemm_tile.grouped_64" in launched and "attention.tiles" in launched
        assert "attention.direct" in launched or "attention.partial" in launched
        assert "route_topk" in launched and "moe_align" in launched      # above 16 rows the routing is two launches
    else:
        # head size 24 on pages of 8 is the universal attention's; the products (K = 96, 192, 48) stay on the matrix cores
        assert "attention.generic" in launched and not {"gemm_generic", "gemm_generic.grouped"} & set(launched)


REAL_LAYER = dict(vocab_size=200064, hidden_size=3072, num_hidden_layers=1, num_attention_heads=48, num_key_value_heads=8, head_dim=128,
                  rotary_dim=64, rope_theta=5e6, rms_norm_eps=1e-6, num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536,
                  routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=4096)


@pytest.fixture(scope="module")
def real_layer_engine():
    """One layer of the real sizes (all 256 experts, the whole vocabulary), weights generated on the device."""
    from llmx_amd import Engine, MiniMaxM3Config, RandomInit
    return Engine.from_random(MiniMaxM3Config(**REAL_LAYER), RandomInit(seed=5, std=0.02, norm_std=0.05, bias_range=0.05), dtype="bfloat16",
                              kv_tokens=24576, page_tokens=16, max_requests=65)


@pytest.mark.parametrize("n_requests", [17, 33, 64])
def test_many_requests_decoded_together_at_the_real_sizes(real_layer_engine, n_requests):
    """The steps a benchmark of batch 16, 32 and 64 times, checked: every kernel form such a step takes was launched and
    every request's logits over the whole vocabulary are those of its run alone."""
    launched = check_decoding_together(real_layer_engine, REAL_LAYER["vocab_size"], n_requests, 16, seed=1000 + n_requests)
    assert not set(launched) & UNIVERSAL, f"the bfloat16 engine fell to {sorted(set(launched) & UNIVERSAL)}"
    # dense products of 17 to 64 rows: tiles of 128 features with K's runs in workgroups of their own
    assert "gemm_tile.runs_apart" in launched and "gemm_skinny.two_strips" not in launched, sorted(launched)
    # routed products above 16 token rows and the head above 16 rows: the tiled kernels
    assert "gemm_tile.grouped_64" in launched and ("gemm_tile.wide" in launched or "gemm_tile.64" in launched)
    assert "route_topk" in launched and "moe_align" in launched and "route_topk_align" not in launched
    # decoding rows: contexts shared out over items and merged, until the rows alone are 512 items (64 rows x 8 KV heads)
    if n_requests < 64:
        assert "attention.partial" in launched and "attention.merge" in launched
    else:
        assert "attention.direct" in launched and "attention.partial" not in launched and "attention.merge" not in launched
    assert "attention.tiles128" in launched
    assert "gemm_f32.skinny" in launched


def test_a_long_portion_beside_decoding_requests_equals_each_alone(real_layer_engine):
    """The step a scheduler issues under load: 512 tokens of one prompt beside the next tokens of 8 decoding requests."""
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    engine = real_layer_engine
    vocab = REAL_LAYER["vocab_size"]
    rng = random.Random(77)
    lengths = [700, 33, 1023, 150, 5, 895, 260, 64]
    prompts = [[rng.randrange(vocab) for _ in range(n)] for n in lengths]
    nexts = [rng.randrange(vocab) for _ in lengths]
    long_prompt = [rng.randrange(vocab) for _ in range(300 + 512)]
    for i, p in enumerate(prompts):
        engine.add_request(i)
        engine.step([StepEntry(i, p, [])])
    engine.add_request("long")
    engine.step([StepEntry("long", long_prompt[:300], [])])
    want_long = [0, 17, 255, 256, 511]
    ops.take_launches()
    mixed = engine.step([StepEntry(i, [nexts[i]], [0]) for i in range(4)] + [StepEntry("long", long_prompt[300:], want_long)]
                        + [StepEntry(i, [nexts[i]], [0]) for i in range(4, 8)]).clone()
    launched = ops.take_launches()
    for i in range(8):
        engine.end_request(i)
    engine.end_request("long")
    assert not set(launched) & UNIVERSAL
    # 520 rows: dense products on tiles, 4,160 pairs grouped on tiles chosen on the device, prompt tiles beside decoding items
    assert "gemm_tile.wide" in launched or "gemm_tile.64" in launched
    assert "gemm_tile.grouped_64" in launched and "attention.tiles128" in launched
    assert "attention.partial" in launched or "attention.direct" in launched or "attention.split4" in launched
    order = [0, 1, 2, 3, "long", 4, 5, 6, 7]
    row = 0
    for rid in order:
        if rid == "long":
            engine.add_request("alone")
            want = engine.step([StepEntry("alone", long_prompt, [300 + w for w in want_long])]).clone()
            engine.end_request("alone")
            n = len(want_long)
        else:
            want = alone(engine, prompts[rid], [nexts[rid]])
            n = 1
        assert torch.equal(mixed[row:row + n], want), f"request {rid!r} in the mixed step differs from its run alone"
        row += n
    assert engine.cache.pages_in_use() == 0
