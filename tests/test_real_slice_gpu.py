"""The real layer sizes (hidden 3072, 48 query / 8 KV heads of 128, rotary 64, 256 experts top-8 of intermediate 1536,
vocabulary 200,064) with random weights: against the plain implementation, and the cuttings against each other.

Method of the reference's own parity runs (/root/reference/tests/minimax.py:63-90: the module's logits beside a
straightforward forward pass; /root/reference/tools/model_logits.cpp:82-109: the same tokens whole and step by step).
Weights are generated on the device from (seed, tensor name); the plain implementation reads the same tensors by name,
copied to the host as it touches them (only the experts a row picked), and a sample far into the largest tensor is
checked against the generator's formula written out here.
"""

from __future__ import annotations

import math
import random

import pytest
import torch

import plain_model
from helpers import PICK_SLACK, ROUTER_TOL, RoutingRecorder, portions

pytestmark = pytest.mark.gpu

REAL = dict(vocab_size=200064, hidden_size=3072, num_attention_heads=48, num_key_value_heads=8, head_dim=128, rotary_dim=64, rope_theta=5e6,
            rms_norm_eps=1e-6, num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536, routed_scaling_factor=1.0,
            norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=4096)


def real_engine(layers, dtype, kv_tokens, max_requests=4, seed=0, bias_range=0.0, keep=None):
    from llmx_amd import Engine, MiniMaxM3Config, RandomInit
    cfg = MiniMaxM3Config(num_hidden_layers=layers, **REAL)
    init = RandomInit(seed=seed, std=0.02, norm_std=0.05 if keep is not None else 0.0, bias_range=bias_range)
    return Engine.from_random(cfg, init, dtype=dtype, kv_tokens=kv_tokens, page_tokens=16, max_requests=max_requests, tensors_out=keep), cfg, init


class HostView:
    """The device tensors by name for the plain implementation: a small tensor comes to the host whole at its first
    use; a tensor of experts is indexed by expert and brings only that expert."""

    class Experts:
        def __init__(self, t):
            self.t, self.got = t, {}

        def __getitem__(self, e):
            if e not in self.got:
                self.got[e] = self.t[e].cpu()
            return self.got[e]

    class Rows:
        def __init__(self, t):
            self.t = t

        def __getitem__(self, rows):
            return self.t[torch.as_tensor(rows, device=self.t.device)].cpu()

    def __init__(self, tensors):
        self.tensors, self.got = tensors, {}

    def __getitem__(self, name):
        if name not in self.got:
            t = self.tensors[name]
            if t.dim() == 3:
                self.got[name] = HostView.Experts(t)
            elif name == "model.embed_tokens.weight":
                self.got[name] = HostView.Rows(t)
            else:
                self.got[name] = t.cpu()
        return self.got[name]


def generator_values(seed, name, start, count, std):
    """N(0, std) values start .. start + count of tensor `name`: the formula the fill kernel documents (FNV-1a of the name and
    the seed mixed into a key; element i from mix64(key + i * golden): two 24-bit uniforms, Box-Muller), written out anew."""
    M = (1 << 64) - 1

    def mix(x):
        x ^= x >> 30
        x = (x * 0xBF58476D1CE4E5B9) & M
        x ^= x >> 27
        x = (x * 0x94D049BB133111EB) & M
        return x ^ (x >> 31)

    h = 0xCBF29CE484222325
    for b in name.encode():
        h = ((h ^ b) * 0x100000001B3) & M
    key = mix((seed * 0x9E3779B97F4A7C15 + h) & M)
    out = []
    for i in range(start, start + count):
        v = mix((key + i * 0x9E3779B97F4A7C15) & M)
        u1 = ((v >> 40) + 1) * 2.0 ** -24
        u2 = ((v >> 8) & 0xFFFFFF) * 2.0 ** -24
        out.append(std * math.sqrt(-2.0 * math.log(u1)) * math.cos(6.2831853 * u2))
    return torch.tensor(out, dtype=torch.float64)


def run_cuts(engine, rid, tokens, cuts, want_from=0):
    """Feeds tokens[a:b] for each cut; returns the logits of positions >= want_from."""
    from llmx_amd.engine import StepEntry
    engine.add_request(rid)
    rows = []
    for a, b in cuts:
        want = [p - a for p in range(max(a, want_from), b)]
        out = engine.step([StepEntry(rid, tokens[a:b], want)])
        if want:
            rows.append(out.clone())
    engine.end_request(rid)
    return torch.cat(rows)


def run_mixed(engine, seqs, decode_tail, sizes, want_from):
    """All sequences live in turn through an engine that holds `engine.max_requests` of them: each step takes a portion of
    changing size of those still in their prompt beside one token of those in their last `decode_tail` tokens."""
    from llmx_amd.engine import StepEntry
    waiting, live = list(seqs), []
    at = {i: 0 for i in seqs}
    rows = {i: [] for i in seqs}
    step_no, reused = 0, set()
    seen_pages = {}
    while waiting or live:
        while waiting and len(live) < engine.max_requests:
            i = waiting.pop(0)
            engine.add_request(("mix", i))
            live.append(i)
        entries, spans = [], []
        for slot, i in enumerate(live):
            n = len(seqs[i])
            k = 1 if at[i] >= n - decode_tail else min(sizes[(step_no + slot) % len(sizes)], n - decode_tail - at[i])
            want = [p - at[i] for p in range(max(at[i], want_from[i]), at[i] + k)]
            entries.append(StepEntry(("mix", i), seqs[i][at[i]:at[i] + k], want))
            spans.append((i, len(want)))
            at[i] += k
        out = engine.step(entries)
        r = 0
        for i, nw in spans:
            if nw:
                rows[i].append(out[r:r + nw].clone())
            r += nw
            for page in engine.cache.table(("mix", i), 0):
                if seen_pages.setdefault(page, i) != i:
                    reused.add(page)
        for i in list(live):
            if at[i] == len(seqs[i]):
                engine.end_request(("mix", i))
                live.remove(i)
        step_no += 1
    assert engine.cache.pages_in_use() == 0
    return {i: torch.cat(rows[i]) for i in seqs}, reused


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_real_layers_against_the_plain_implementation(dtype):
    """Two layers at the real sizes, 256 experts top-8 and the 200,064-row head inside the engine, four sequences of 41 to
    78 tokens: the logits lie within 3e-5 (float32; 2e-2 in bfloat16) of the float64 plain implementation, relative to
    the largest logit; in float32 the picks are the plain router's own; whole prompts, the last tokens one by one,
    portions of 7, 2 and 13 tokens and a mix through a pool that is used again give the same bits."""
    rng = random.Random(3)
    lengths = [41, 57, 66, 78]
    seqs = {i: [rng.randrange(REAL["vocab_size"]) for _ in range(n)] for i, n in enumerate(lengths)}
    tensors = {}
    # three of the four requests fit the pool at a time: pages are handed out again in the mix
    engine, cfg, init = real_engine(2, dtype, kv_tokens=64 + 80 + 80, max_requests=3, seed=7, bias_range=0.05, keep=tensors)
    rounded = dtype == "bfloat16"

    # the device's weights are the generator's: a sample 2.4e9 elements into the largest tensor, and the head's last row
    name = "model.layers.1.mlp.experts.gate_up_proj"
    X, F2, E = tensors[name].shape
    start = 255 * F2 * E + 1234567
    # float32 values agree to the last places of logf and cosf (1e-7).  A bfloat16 value is the device's float32 value
    # rounded: it must be the bfloat16 rounding of a float32 value within those last places of the one computed here,
    # that is of its lower or its upper end (the two differ only where the value lies on a rounding boundary)
    def close(got, want):
        if not rounded:
            return float((got - want).abs().max()) < 1e-7
        slack = want.abs() * 3e-7 + 1e-9
        ends = [(want + d).float().to(torch.bfloat16).double() for d in (-slack, slack)]
        return bool(((got == ends[0]) | (got == ends[1])).all())
    got = tensors[name].view(-1)[start:start + 64].double().cpu()
    assert close(got, generator_values(7, name, start, 64, 0.02))
    last_row = tensors["lm_head.weight"][-1, :64].double().cpu()
    assert close(last_row, generator_values(7, "lm_head.weight", (REAL["vocab_size"] - 1) * E, 64, 0.02))

    recorder = RoutingRecorder(2)
    engine.observer = recorder
    whole = {i: run_cuts(engine, ("whole", i), t, [(0, len(t))]) for i, t in seqs.items()}
    engine.observer = None
    host = HostView(tensors)
    config = cfg.to_json()
    k = REAL["num_experts_per_tok"]
    for i, t in seqs.items():
        n = len(t)
        picks, router = recorder.of(("whole", i), n), recorder.logits_of(("whole", i), n)
        want, routing = plain_model.forward(config, host, t, torch.float64, torch.bfloat16 if rounded else None, return_routing=True,
                                            picks=picks if rounded else None)
        for layer, (ids, _, keys, z) in enumerate(routing):
            if not rounded:
                assert torch.equal(ids, picks[layer]), f"sequence {i}, layer {layer}: the float32 router picked other experts than the plain router"
            # every row's picks are the best k keys of the engine's own logits, and those logits are the plain ones
            bias = host[f"model.layers.{layer}.mlp.gate.e_score_correction_bias"].float()
            own = (1.0 / (1.0 + torch.exp(-router[layer].float())) + bias).double()
            kth = torch.sort(own, dim=-1, descending=True).values[:, k - 1]
            assert (torch.gather(own, 1, picks[layer]) >= kth[:, None] - PICK_SLACK).all()
            assert float((router[layer].double() - z).abs().max()) <= ROUTER_TOL[rounded] * max(1.0, float(z.abs().max()))
        err, scale = float((whole[i].double().cpu() - want).abs().max()), float(want.abs().max())
        assert err <= (3e-5 if not rounded else 2e-2) * scale, f"sequence {i} ({n} tokens, {dtype}): max error {err:.3e} against the largest logit {scale:.3e}"

    for i, t in seqs.items():
        n = len(t)
        tail = min(32, n - 1)
        one_by_one = run_cuts(engine, ("dec", i), t, [(0, n - tail)] + [(p, p + 1) for p in range(n - tail, n)])
        assert torch.equal(one_by_one, whole[i]), f"sequence {i}: the last {tail} tokens one by one differ from the whole prompt"
        cut = run_cuts(engine, ("por", i), t, portions(n, sizes=(7, 2, 13)))
        assert torch.equal(cut, whole[i]), f"sequence {i}: portions of 7, 2 and 13 tokens differ from the whole prompt"
    mixed, reused = run_mixed(engine, seqs, decode_tail=8, sizes=(7, 2, 13, 5), want_from={i: 0 for i in seqs})
    assert reused, "the pool held every request at once: no page was used again"
    for i in seqs:
        assert torch.equal(mixed[i], whole[i]), f"sequence {i} in the mix differs from its run alone"
    del engine, tensors, host
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,layers", [("float32", 8), ("bfloat16", 24)], ids=["float32-8-layers", "bfloat16-24-layers"])
def test_real_slice_cuttings_agree_bit_for_bit(dtype, layers):
    """The slices the benchmark runs (8 layers in float32: 122 GB of weights; 24 layers in bfloat16: 179 GB): four sequences
    of 300 to 1,000 tokens whole, with the last 32 tokens one by one, in portions of 64 and mixed, four live with
    portions of some beside decoded tokens of others.  The logits of each sequence's last 40 positions must agree bit
    for bit (a router's near-tie that fell differently under two cuttings would change an expert and, through the
    layers, several percent of the largest logit)."""
    lengths = [300, 517, 764, 1000]
    rng = random.Random(11)
    seqs = {i: [rng.randrange(REAL["vocab_size"]) for _ in range(n)] for i, n in enumerate(lengths)}
    engine, _, _ = real_engine(layers, dtype, kv_tokens=sum(-(-n // 64) * 64 for n in lengths))
    tail = {i: len(t) - 40 for i, t in seqs.items()}
    whole = {i: run_cuts(engine, ("whole", i), t, [(0, len(t))], tail[i]) for i, t in seqs.items()}
    assert all(bool(torch.isfinite(g).all()) and g.shape[0] == 40 for g in whole.values())
    for i, t in seqs.items():
        n = len(t)
        got = run_cuts(engine, ("dec", i), t, [(0, n - 32)] + [(p, p + 1) for p in range(n - 32, n)], tail[i])
        assert torch.equal(got, whole[i]), f"sequence {i}: the last 32 tokens one by one differ from the whole prompt"
        got = run_cuts(engine, ("por", i), t, [(p, min(p + 64, n)) for p in range(0, n, 64)], tail[i])
        assert torch.equal(got, whole[i]), f"sequence {i}: portions of 64 differ from the whole prompt"
    mixed, _ = run_mixed(engine, seqs, decode_tail=16, sizes=(64, 7, 128, 2, 33), want_from=tail)
    for i in seqs:
        assert torch.equal(mixed[i], whole[i]), f"sequence {i} in the mix differs from its run alone"
    del engine
    torch.cuda.empty_cache()
