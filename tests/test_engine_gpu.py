"""The engine against the plain implementation, under every way of cutting the same tokens into steps.

For each tiny configuration and both dtypes: each request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; and mixed, up to four live requests, portions of some
beside decoded tokens of others, with so few pages that they are used again.  In both dtypes the cuttings must agree
with each other bit for bit (every kernel's per-row arithmetic is independent of the batch); with the plain
implementation they agree within F32_TOL in float32 and, rounded at the same places, within BF16_TOL in bfloat16.
"""

from __future__ import annotations

import pytest
import torch

import helpers
from helpers import TINY, RoutingRecorder, model_folder, plain_logits, plain_logits_with_picks, portions, tokens_for

pytestmark = pytest.mark.gpu

# Bounds on |engine - plain| over all logits, relative to the largest |logit| of the sequence.
# float32: the engine sums in float32 in its own order, the plain implementation in float64.
F32_TOL = 2e-5
# bfloat16: both round at the same places; what is left are float32 sums of bfloat16 products whose last-bit
# differences flip a bfloat16 rounding (2^-8 relative) of single activations here and there.  Such a flip can also
# turn a router's near-tie (the tiny models' closest keys lie 1e-5 apart), so in bfloat16 the plain implementation is
# given the engine's picks, after checking in every row that they are the k best keys of the engine's own router logits
# and that those logits are the plain ones within their noise (helpers.plain_logits_with_picks).
BF16_TOL = 2e-2

LENGTHS = {"A": (5, 17, 32, 75), "B": (1, 9, 23, 40, 67), "A16": (5, 17, 32, 75)}


def make_engine(name, dtype, kv_tokens=1024, max_requests=8):
    from llmx_amd.engine import Engine
    return Engine.load(model_folder(name), dtype=dtype, kv_tokens=kv_tokens, page_tokens=TINY[name][2], max_requests=max_requests)


def watch(engine, name, dtype):
    """In bfloat16 the engine's expert picks are recorded for the comparison; float32 must pick as the plain router does."""
    engine.observer = RoutingRecorder(TINY[name][0]["num_hidden_layers"]) if dtype == "bfloat16" else None
    return engine


@pytest.fixture(scope="module", params=[("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16"), ("A16", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def setup(request):
    name, dtype = request.param
    return name, dtype, watch(make_engine(name, dtype), name, dtype)


def run_whole(engine, rid, tokens):
    from llmx_amd.engine import StepEntry
    engine.add_request(rid)
    logits = engine.step([StepEntry(rid, tokens, list(range(len(tokens))))]).clone()
    engine.end_request(rid)
    return logits.cpu()


def run_cut(engine, rid, tokens, cuts):
    from llmx_amd.engine import StepEntry
    engine.add_request(rid)
    rows = []
    for a, b in cuts:
        rows.append(engine.step([StepEntry(rid, tokens[a:b], list(range(b - a)))]).clone())
    engine.end_request(rid)
    return torch.cat(rows).cpu()


def check_against_plain(name, dtype, length, seed, got, engine=None, rid=None):
    if dtype == "bfloat16":
        want = plain_logits_with_picks(name, tokens_for(name, length, seed), engine.observer.of(rid, length),
                                       engine_logits=engine.observer.logits_of(rid, length))
    else:
        want = plain_logits(name, length, seed, False)
    tol = F32_TOL if dtype == "float32" else BF16_TOL
    scale = float(want.abs().max())
    err = float((got.double() - want).abs().max())
    assert err <= tol * scale, f"{name} {dtype} length {length}: max error {err:.3e} against scale {scale:.3e}"


def test_whole_alone(setup):
    name, dtype, engine = setup
    for length in LENGTHS[name]:
        tokens = tokens_for(name, length, 0)
        got = run_whole(engine, "w", tokens)
        assert got.shape == (length, TINY[name][0]["vocab_size"])
        assert torch.isfinite(got).all()
        check_against_plain(name, dtype, length, 0, got, engine, "w")
    assert engine.cache.pages_in_use() == 0


def test_last_32_one_by_one(setup):
    name, dtype, engine = setup
    length = 67 if name == "B" else 75
    tokens = tokens_for(name, length, 0)
    whole = run_whole(engine, "w", tokens)
    cuts = [(0, length - 32)] + [(i, i + 1) for i in range(length - 32, length)]
    got = run_cut(engine, "d", tokens, cuts)
    check_against_plain(name, dtype, length, 0, got, engine, "d")
    assert torch.equal(got, whole), f"decoding one by one differs from the whole prompt in {dtype}"


def test_portions_of_changing_size(setup):
    name, dtype, engine = setup
    length = 67 if name == "B" else 75
    tokens = tokens_for(name, length, 0)
    whole = run_whole(engine, "w", tokens)
    got = run_cut(engine, "p", tokens, portions(length))
    check_against_plain(name, dtype, length, 0, got, engine, "p")
    assert torch.equal(got, whole), f"portions differ from the whole prompt in {dtype}"


def test_first_tokens(setup):
    """The first tokens of a sequence: lengths 1 and 2, and the first rows of a longer one."""
    name, dtype, engine = setup
    for length in (1, 2, 3):
        tokens = tokens_for(name, 67 if name == "B" else 75, 0)[:length]
        got = run_whole(engine, "f", tokens)
        if dtype == "bfloat16":
            want = plain_logits_with_picks(name, tokens, engine.observer.of("f", length), engine_logits=engine.observer.logits_of("f", length))
        else:
            want = plain_logits(name, 67 if name == "B" else 75, 0, False)[:length]
        tol = F32_TOL if dtype == "float32" else BF16_TOL
        assert float((got.double() - want).abs().max()) <= tol * float(want.abs().max())


def test_truncate_takes_a_request_back_to_a_prefix(setup):
    """A request is taken back to 41 of its tokens (inside a page) and goes on with other tokens: the logits are those
    of a fresh run of the new sequence, bit for bit, and the pages beyond the prefix went back to the pool."""
    from llmx_amd.engine import StepEntry
    name, dtype, engine = setup
    page = TINY[name][2]
    length = 67 if name == "B" else 75
    tokens, other = tokens_for(name, length, 0), tokens_for(name, length, 9)
    joined = tokens[:41] + other[41:]
    whole, whole_joined = run_whole(engine, "w", tokens), run_whole(engine, "w", joined)
    every = lambda t: list(range(len(t)))
    engine.add_request("t")
    assert torch.equal(engine.step([StepEntry("t", tokens, every(tokens))]).cpu(), whole)
    assert engine.cache.pages_in_use() == -(-length // page)
    engine.truncate("t", 41)
    assert engine.length("t") == 41 and engine.cache.pages_in_use() == -(-41 // page)
    assert torch.equal(engine.step([StepEntry("t", other[41:], every(other[41:]))]).cpu(), whole_joined[41:])
    engine.truncate("t", 0)
    assert engine.cache.pages_in_use() == 0
    assert torch.equal(engine.step([StepEntry("t", tokens[:30], every(tokens[:30]))]).cpu(), whole[:30])
    from llmx_amd.cache import CacheLogicError
    with pytest.raises(CacheLogicError, match="cannot be taken back to 31"):
        engine.truncate("t", 31)
    engine.end_request("t")
    assert engine.cache.pages_in_use() == 0


def test_the_router_reads_unrounded_rows_in_bfloat16():
    """The router's logits come from the float32 normed rows, not from their bfloat16 roundings
    (/root/reference/src/backends/backend.hpp:943-947: the router's product is F32 whatever the step's type).  Eight
    one-token requests in one step: with a single key the softmax weight is exactly 1, so everything before the router is
    the plain implementation's arithmetic up to the order of float32 sums, and the engine's logits can be told apart from
    the logits a router reading rounded rows would give."""
    import plain_model as pm
    from helpers import INIT_B, TINY_B, plain
    from llmx_amd.engine import StepEntry
    helpers.TINY["B1"] = (dict(TINY_B, num_hidden_layers=1), INIT_B, 8)
    engine = make_engine("B1", "bfloat16")
    engine.observer = RoutingRecorder(1)
    tokens = tokens_for("B1", 8, 3)
    for i in range(8):
        engine.add_request(i)
    engine.step([StepEntry(i, [t], []) for i, t in enumerate(tokens)])
    z_engine = torch.stack([engine.observer.logits_of(i, 1)[0][0] for i in range(8)]).double()
    cfg, w = plain("B1")
    bf, eps, p = torch.bfloat16, cfg["rms_norm_eps"], "model.layers.0."
    z_wide, z_rounded = [], []
    for t in tokens:
        x = w["model.embed_tokens.weight"].double()[[t]]
        x = x + pm.attention_layer(pm.rms_norm(x, w[p + "input_layernorm.weight"].double(), eps), [0], w, p + "self_attn.", cfg, bf)
        h = pm.rms_norm(x, w[p + "post_attention_layernorm.weight"].double(), eps)
        z_wide.append(h @ w[p + "mlp.gate.weight"].double().T)
        z_rounded.append(pm._rounded(h, bf) @ w[p + "mlp.gate.weight"].double().T)
    z_wide, z_rounded = torch.cat(z_wide), torch.cat(z_rounded)
    apart = float((z_rounded - z_wide).abs().max())
    assert apart > 1e-4 * float(z_wide.abs().max())                     # the two readings can be told apart here
    assert float((z_engine - z_wide).abs().max()) < 0.02 * apart        # and the engine's is the unrounded one
    assert float((z_engine - z_rounded).abs().max()) > 0.5 * apart


MIXED_LENGTHS = [40, 23, 67, 9, 31, 52]
MIXED_SEEDS = [1, 2, 3, 4, 5, 6]


def run_mixed(name, dtype):
    """Six requests through a pool for four: up to four live, portions of some beside decoded tokens of others, some left
    out of a step.  Returns the engine, the prompts and each request's logits [length, vocab] as the steps gave them."""
    from llmx_amd.engine import StepEntry
    page = TINY[name][2]
    lengths, seeds = MIXED_LENGTHS, MIXED_SEEDS
    # four live requests of at most 67 tokens: pages for 4 * 72 tokens, far fewer than all six hold together
    engine = watch(make_engine(name, dtype, kv_tokens=4 * (-(-67 // page) * page), max_requests=4), name, dtype)
    toks = [tokens_for(name, n, s) for n, s in zip(lengths, seeds)]
    got = {i: [] for i in range(len(lengths))}
    at = {i: 0 for i in range(len(lengths))}
    waiting = list(range(len(lengths)))
    live = []
    used_pages = set()
    step_no = 0
    while waiting or live:
        while waiting and len(live) < 4:
            i = waiting.pop(0)
            engine.add_request(i)
            live.append(i)
        entries = []
        for slot, i in enumerate(live):
            n_left = lengths[i] - at[i]
            prefill_end = lengths[i] - 8          # the last 8 tokens of every request are decoded one by one
            if at[i] >= prefill_end:
                n = 1
            else:
                n = min((5, 2, 11, 3)[(step_no + slot) % 4], prefill_end - at[i])
            if (step_no + i) % 5 == 4 and len(live) > 1:
                continue                           # a request may be left out of a step and go on later
            entries.append(StepEntry(i, toks[i][at[i]:at[i] + n], list(range(n))))
        if entries:
            logits = engine.step(entries).clone().cpu()
            row = 0
            for e in entries:
                n = len(e.tokens)
                got[e.request].append(logits[row:row + n])
                row += n
                at[e.request] += n
                for g in range(len(engine.cache.groups)):
                    used_pages.update(engine.cache.table(e.request, g))
        for i in list(live):
            if at[i] == lengths[i]:
                engine.end_request(i)
                live.remove(i)
        step_no += 1
        assert step_no < 1000
    assert engine.cache.pages_in_use() == 0
    total_pages = sum(-(-n // page) for n in lengths)
    assert len(used_pages) < total_pages, "the pool was large enough that no page was used again"
    return engine, toks, [torch.cat(got[i]) for i in range(len(lengths))]


def test_mixed_requests_with_page_reuse(setup):
    """Up to four live requests; portions of some beside decoded tokens of others; the pool is so small that pages
    freed by finished requests are handed out again."""
    name, dtype, _ = setup
    engine, toks, mixed = run_mixed(name, dtype)
    alone = make_engine(name, dtype)
    for i, (n, s) in enumerate(zip(MIXED_LENGTHS, MIXED_SEEDS)):
        check_against_plain(name, dtype, n, s, mixed[i], engine, i)
        assert torch.equal(mixed[i], run_whole(alone, "w", toks[i])), f"request {i} in the mix differs from its run alone"


def test_long_decoding(setup):
    """A short prompt, then 200 tokens decoded one by one across many page edges."""
    name, dtype, engine = setup
    length = 8 + 200
    tokens = tokens_for(name, length, 7)
    cuts = [(0, 8)] + [(i, i + 1) for i in range(8, length)]
    got = run_cut(engine, "l", tokens, cuts)
    check_against_plain(name, dtype, length, 7, got, engine, "l")


@pytest.mark.parametrize("name,dtype", [("A", "bfloat16"), ("B", "float32"), ("A16", "bfloat16")])
def test_decode_steps_replayed_as_graphs_equal_eager_steps(name, dtype):
    """Steps of single decoded tokens are replayed as HIP graphs once their shape has been seen.  Every replay gives the
    bits of an engine that never records a graph, with prompts of other requests (eager work), synchronisations, page
    edges and a change of the batch between the replays."""
    from llmx_amd.engine import Engine, StepEntry
    page = TINY[name][2]
    engines = [Engine.load(model_folder(name), dtype=dtype, kv_tokens=1024, page_tokens=page, max_requests=8, graphs=g) for g in (True, False)]
    assert engines[0].graphs and not engines[1].graphs
    prompts = {"a": tokens_for(name, 9, 1), "b": tokens_for(name, 30, 2), "c": tokens_for(name, 3, 3)}
    extra = tokens_for(name, 70, 4)
    last = {}
    for eng in engines:
        for rid, toks in prompts.items():
            eng.add_request(rid)
            last[rid] = eng.step([StepEntry(rid, toks, [len(toks) - 1])]).argmax(dim=1).item()
    live = ["a", "b", "c"]
    nxt = dict(last)
    for i in range(60):
        outs = []
        for eng in engines:
            if i == 12:
                eng.add_request("x")
                eng.step([StepEntry("x", extra[:33], [])])        # another request's prompt between the replays
                torch.cuda.synchronize()
            if i == 30:
                eng.step([StepEntry("x", extra[33:], [36])])
                eng.end_request("x")
            outs.append(eng.step([StepEntry(rid, [nxt[rid]], [0]) for rid in live]).clone())
        assert torch.equal(outs[0], outs[1]), f"step {i}: the replayed step differs from the eager one"
        picks = outs[0].argmax(dim=1).tolist()
        nxt = {rid: p for rid, p in zip(live, picks)}
        if i == 40:
            for eng in engines:
                eng.end_request("b")
            live = ["a", "c"]
            nxt.pop("b")
    assert engines[0].graph_replays >= 40 and engines[1].graph_replays == 0


@pytest.mark.parametrize("name,dtype,prompt_len", [("A", "bfloat16", 250), ("A16", "bfloat16", 885), ("B", "float32", 505)])
def test_graph_replays_across_the_edges_their_key_exists_for(name, dtype, prompt_len):
    """Decoding crosses the sizes a recorded step is keyed by: the block table's width (64 pages: 256 tokens on pages of
    4, 512 on pages of 8), the attention plan's segment count (896 tokens, where the split contexts' partial results get
    more slots), and scratch storage that moves because another request's larger portion ran between two replays (the
    recorded graphs are dropped and recorded again).  Every step equals an engine that records nothing."""
    from llmx_amd.engine import Engine, StepEntry
    page = TINY[name][2]
    engines = [Engine.load(model_folder(name), dtype=dtype, kv_tokens=2048, page_tokens=page, max_requests=4, graphs=g) for g in (True, False)]
    prompt, extra = tokens_for(name, prompt_len, 21), tokens_for(name, 400, 22)
    nxt = None
    for eng in engines:
        eng.add_request("a")
        for s in range(0, prompt_len, 200):        # portions of 200: the larger portion below makes scratch storage grow
            part = prompt[s:s + 200]
            out = eng.step([StepEntry("a", part, [len(part) - 1])])
        nxt = int(out.argmax(dim=1))
    replays_before_growth = None
    for i in range(40):
        outs = []
        for eng in engines:
            if i == 20:
                eng.add_request("x")
                eng.step([StepEntry("x", extra, [])])
                eng.end_request("x")
            outs.append(eng.step([StepEntry("a", [nxt], [0])]).clone())
        if i == 19:
            replays_before_growth = engines[0].graph_replays
        assert torch.equal(outs[0], outs[1]), f"step {i} (context {prompt_len + i + 1}): the replayed step differs from the eager one"
        nxt = int(outs[0].argmax(dim=1))
    assert replays_before_growth >= 10 and engines[0].graph_replays >= replays_before_growth + 10 and engines[1].graph_replays == 0


def test_a_folder_with_per_expert_tensors_gives_the_logits_of_the_fused_folder(tmp_path):
    """experts.N.{gate,up,down}_proj.weight instead of the fused tensors: the loader fuses them on the way to the device."""
    import json, shutil
    from safetensors import safe_open
    from llmx_amd.engine import Engine, StepEntry
    from llmx_amd.weights import write_safetensors
    src = model_folder("B")
    split = {}
    with safe_open(f"{src}/model.safetensors", framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            if name.endswith("experts.gate_up_proj"):
                half = t.shape[1] // 2
                for e in range(t.shape[0]):
                    split[name[:-len("gate_up_proj")] + f"{e}.gate_proj.weight"] = t[e, :half].clone()
                    split[name[:-len("gate_up_proj")] + f"{e}.up_proj.weight"] = t[e, half:].clone()
            elif name.endswith("experts.down_proj"):
                for e in range(t.shape[0]):
                    split[name[:-len("down_proj")] + f"{e}.down_proj.weight"] = t[e].clone()
            else:
                split[name] = t
    shutil.copy(f"{src}/config.json", tmp_path / "config.json")
    write_safetensors(tmp_path / "model.safetensors", split)
    tokens = tokens_for("B", 23, 4)
    outs = []
    for folder in (src, str(tmp_path)):
        eng = Engine.load(folder, dtype="bfloat16", kv_tokens=64, page_tokens=8, max_requests=1)
        eng.add_request(0)
        outs.append(eng.step([StepEntry(0, tokens, list(range(23)))]).clone())
    assert torch.equal(outs[0], outs[1])


def test_refusals_leave_nothing_behind(setup):
    from llmx_amd.engine import StepEntry, StepError
    name, dtype, engine = setup
    vocab = TINY[name][0]["vocab_size"]
    engine.add_request("r")
    before = engine.cache.pages_in_use()
    with pytest.raises(StepError, match="outside the embedding"):
        engine.step([StepEntry("r", [1, vocab], [0])])
    with pytest.raises(StepError, match="twice"):
        engine.step([StepEntry("r", [1], [0]), StepEntry("r", [2], [0])])
    with pytest.raises(StepError, match="not open"):
        engine.step([StepEntry("nobody", [1], [0])])
    with pytest.raises(StepError, match="no tokens"):
        engine.step([StepEntry("r", [], [])])
    with pytest.raises(StepError, match="empty"):
        engine.step([])
    assert engine.cache.pages_in_use() == before and engine.length("r") == 0
    engine.end_request("r")


# ---------------------------------------------------------------------------
# One layer at the real layer widths (hidden 3072, 48 query / 8 KV heads of 128, rotary 64, theta 5e6, expert
# intermediate 1536, top-8) with fewer experts and a small vocabulary, so that the plain implementation stays fast:
# the products, the attention and the routing run at the K, N and head sizes of the real model.
WIDE = dict(vocab_size=1000, hidden_size=3072, num_hidden_layers=1, num_attention_heads=48, num_key_value_heads=8, head_dim=128,
            rotary_dim=64, rope_theta=5e6, rms_norm_eps=1e-6, num_local_experts=16, num_experts_per_tok=8, intermediate_size=1536,
            routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=4096)


@pytest.fixture(scope="module")
def wide_folder(tmp_path_factory):
    from llmx_amd import MiniMaxM3Config, RandomInit
    from llmx_amd.weights.folder import write_random_model
    folder = tmp_path_factory.mktemp("wide")
    write_random_model(folder, MiniMaxM3Config(**WIDE), RandomInit(seed=3, std=0.02, norm_std=0.05, bias_range=0.05))
    return str(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_widths(wide_folder, dtype):
    import plain_model
    from llmx_amd.engine import Engine, StepEntry
    import random
    cfg, w = plain_model.load_folder(wide_folder)
    rng = random.Random(5)
    tokens = [rng.randrange(1000) for _ in range(150)]
    engine = Engine.load(wide_folder, dtype=dtype, kv_tokens=512, page_tokens=16, max_requests=2)
    recorder = RoutingRecorder(1)
    engine.observer = recorder
    engine.add_request("w")
    whole = engine.step([StepEntry("w", tokens, list(range(150)))]).clone().cpu()
    engine.end_request("w")
    picks = recorder.of("w", 150)
    rounded = torch.bfloat16 if dtype == "bfloat16" else None
    want, routing = plain_model.forward(cfg, w, tokens, torch.float64, rounded, return_routing=True, picks=picks if rounded else None)
    if not rounded:
        assert torch.equal(routing[0][0], picks[0]), "the float32 router picked other experts than the plain router"
    tol = 3e-5 if dtype == "float32" else BF16_TOL
    assert float((whole.double() - want).abs().max()) <= tol * float(want.abs().max())
    # in portions (70 rows take the tiled kernels, 2 and 13 the streaming ones) and token by token at the end
    from llmx_amd import ops
    engine.add_request("p")       # the observer stays set, so no step is recorded as a graph and every launch is counted
    cuts = [(0, 70), (70, 72), (72, 85), (85, 140)] + [(i, i + 1) for i in range(140, 150)]
    rows, launched = [], []
    for a, b in cuts:
        ops.take_launches()
        rows.append(engine.step([StepEntry("p", tokens[a:b], list(range(b - a)))]).clone())
        launched.append(ops.take_launches())
    rows = torch.cat(rows).cpu()
    engine.end_request("p")
    assert torch.equal(rows, whole), f"portions differ from the whole prompt in {dtype}"
    universal = {"gemm_generic", "gemm_generic.grouped", "attention.generic"}
    if dtype == "bfloat16":
        assert not any(universal & set(l) for l in launched), "a bfloat16 step at the real widths fell to the universal kernels"
        assert {"gemm_tile.64", "gemm_tile.grouped_64", "attention.tiles128", "gemm_f32.skinny"} <= set(launched[0])      # 70 rows
        assert {"gemm_skinny", "gemm_skinny.grouped", "route_topk_align"} <= set(launched[1]) and not any(k.startswith("gemm_tile") for k in launched[1])
        assert {"gemm_skinny", "gemm_skinny.grouped"} <= set(launched[2])                                            # 13 rows
        # one row: the norms are formed inside the products, the context's segments go to workgroups of four waves
        assert {"gemm_skinny.normed", "gemm_skinny.grouped_normed", "gemm_f32.normed", "attention.split4", "attention.merge"} <= set(launched[-1])
        assert launched[-1].get("rmsnorm", 0) == 1                      # only the final norm runs as a kernel of its own
    else:
        assert all(universal <= set(l) for l in launched)
        assert not any(k.startswith(("gemm_skinny", "gemm_tile", "attention.")) and k != "attention.generic" for l in launched for k in l)


def test_a_long_portion_takes_the_wide_tiles_and_gives_the_bits_of_short_ones(wide_folder):
    """800 rows at the real layer widths run the dense products on the wide tiles and the routed ones (6,400 pairs) on
    tiles chosen on the device; the same prompt in portions that stay below those sizes gives the same logits bit for bit."""
    from llmx_amd.engine import Engine, StepEntry
    import random
    rng = random.Random(11)
    tokens = [rng.randrange(1000) for _ in range(800)]
    want_rows = list(range(0, 800, 37)) + [799]
    engine = Engine.load(wide_folder, dtype="bfloat16", kv_tokens=2048, page_tokens=16, max_requests=2)
    from llmx_amd import ops
    engine.add_request("w")
    ops.take_launches()
    whole = engine.step([StepEntry("w", tokens, want_rows)]).clone()
    launched = ops.take_launches()
    engine.end_request("w")
    assert bool(torch.isfinite(whole).all())
    # QKV: 7 x 32 wide tiles fill the chip; the output projection (7 x 12) takes 64-row tiles; 6,400 pairs are launched
    # in a 128-row form (wide for K = 3072, four waves for K = 1536) beside the 64-row form, chosen on the device
    assert launched.get("gemm_tile.wide", 0) == 1 and launched.get("gemm_tile.64", 0) == 1
    assert launched.get("gemm_tile.grouped_wide", 0) == 1 and launched.get("gemm_tile.grouped_128", 0) == 1
    assert launched.get("gemm_tile.grouped_64", 0) == 2 and launched.get("attention.tiles128", 0) == 1
    assert not {"gemm_generic", "gemm_generic.grouped", "attention.generic"} & set(launched)
    engine.add_request("p")
    rows = []
    for a, b in [(0, 300), (300, 330), (330, 650), (650, 799), (799, 800)]:
        want = [r - a for r in want_rows if a <= r < b]
        out = engine.step([StepEntry("p", tokens[a:b], want)])
        rows.append(out.clone())
    engine.end_request("p")
    assert torch.equal(torch.cat(rows), whole)
