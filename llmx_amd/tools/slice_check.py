"""Logit equality across cuttings on a random-weight slice with the real layer sizes (too large for the test suite).

    python -m llmx_amd.tools.slice_check --dtype float32 --layers 8      # the 8-layer float32 slice: about 116 GB of weights
    python -m llmx_amd.tools.slice_check --dtype bfloat16 --layers 24    # the 24-layer bfloat16 slice the benchmark runs

Four sequences of 300 to 1,000 seeded random tokens are run (1) each alone and whole, (2) most in one step and the last
32 tokens one by one, (3) in 64-token portions, (4) mixed, up to four live requests with portions of some beside decoded
tokens of others.  Only the logits of each sequence's last 40 positions are compared (a full [1000, 200064] float32
block per cutting would not fit the host comfortably).  The cuttings must agree bit for bit in both dtypes.
"""

from __future__ import annotations

import argparse
import json
import random
import sys
import time


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--dtype", choices=["float32", "bfloat16"], default="float32")
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=200064)
    ap.add_argument("--lengths", default="300,517,764,1000")
    ap.add_argument("--tail", type=int, default=40, help="final positions of each sequence whose logits are compared")
    a = ap.parse_args(argv)

    import torch
    from llmx_amd import Engine, MiniMaxM3Config, RandomInit
    from llmx_amd.engine import StepEntry

    cfg = MiniMaxM3Config(vocab_size=a.vocab, hidden_size=3072, num_hidden_layers=a.layers, num_attention_heads=48, num_key_value_heads=8,
                          head_dim=128, rotary_dim=64, rope_theta=5e6, rms_norm_eps=1e-6, num_local_experts=256, num_experts_per_tok=8,
                          intermediate_size=1536, routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False,
                          max_position_embeddings=4096)
    lengths = [int(x) for x in a.lengths.split(",")]
    rng = random.Random(11)
    seqs = {i: [rng.randrange(a.vocab) for _ in range(n)] for i, n in enumerate(lengths)}
    t0 = time.time()
    engine = Engine.from_random(cfg, RandomInit(seed=0, std=0.02), dtype=a.dtype, kv_tokens=sum(-(-n // 64) * 64 for n in lengths),
                                page_tokens=16, max_requests=4)
    torch.cuda.synchronize()
    print(f"slice_check: {a.layers} layers, {engine.weight_bytes() / 1e9:.1f} GB of weights, made in {time.time() - t0:.1f} s", flush=True)
    tail = a.tail

    def want_of(n, a0, b0):
        """places among tokens [a0, b0) that fall in the sequence's last `tail` positions"""
        return [p - a0 for p in range(max(a0, n - tail), b0)]

    def run_cuts(rid, toks, cuts):
        engine.add_request(rid)
        rows = []
        for a0, b0 in cuts:
            w = want_of(len(toks), a0, b0)
            out = engine.step([StepEntry(rid, toks[a0:b0], w)])
            if w:
                rows.append(out.clone())
        engine.end_request(rid)
        return torch.cat(rows)

    results = {}
    t0 = time.time()
    golden = {i: run_cuts(("whole", i), t, [(0, len(t))]) for i, t in seqs.items()}
    print(f"slice_check: whole prompts in {time.time() - t0:.1f} s", flush=True)
    assert all(torch.isfinite(g).all() for g in golden.values()), "non-finite logits"

    def compare(label, got):
        worst = 0.0
        equal = True
        for i in seqs:
            d = (got[i].double() - golden[i].double()).abs().max().item() / golden[i].abs().max().item()
            worst = max(worst, d)
            equal = equal and torch.equal(got[i], golden[i])
        results[label] = {"bit_equal": equal, "max_relative_difference": worst}
        print(f"slice_check: {label}: bit-equal {equal}, largest relative difference {worst:.3e}", flush=True)

    t0 = time.time()
    compare("last_32_one_by_one", {i: run_cuts(("dec", i), t, [(0, len(t) - 32)] + [(p, p + 1) for p in range(len(t) - 32, len(t))])
                                   for i, t in seqs.items()})
    compare("portions_of_64", {i: run_cuts(("por", i), t, [(p, min(p + 64, len(t))) for p in range(0, len(t), 64)]) for i, t in seqs.items()})
    # mixed: all four live; each step takes a portion of changing size of those still in their prompt and one token of the others
    for i in seqs:
        engine.add_request(("mix", i))
    at = {i: 0 for i in seqs}
    rows = {i: [] for i in seqs}
    step_no = 0
    sizes = (64, 7, 128, 2, 33)
    while any(at[i] < lengths[i] for i in seqs):
        entries, spans = [], []
        for slot, i in enumerate(seqs):
            n = lengths[i]
            if at[i] >= n:
                continue
            decode_from = n - 16
            k = 1 if at[i] >= decode_from else min(sizes[(step_no + slot) % len(sizes)], decode_from - at[i])
            w = want_of(n, at[i], at[i] + k)
            entries.append(StepEntry(("mix", i), seqs[i][at[i]:at[i] + k], w))
            spans.append((i, len(w)))
            at[i] += k
        out = engine.step(entries)
        r = 0
        for i, nw in spans:
            if nw:
                rows[i].append(out[r:r + nw].clone())
            r += nw
        step_no += 1
    for i in seqs:
        engine.end_request(("mix", i))
    compare("mixed_four_live", {i: torch.cat(rows[i]) for i in seqs})
    print(f"slice_check: cuttings in {time.time() - t0:.1f} s", flush=True)
    ok = all(r["bit_equal"] for r in results.values())
    print(json.dumps({"dtype": a.dtype, "layers": a.layers, "lengths": lengths, "results": results, "ok": ok}))
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
