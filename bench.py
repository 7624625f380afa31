"""Decode and prefill throughput of MiniMax-M3 at real layer sizes with random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

A step is one decode step of the whole batch: B requests, each at a context that reaches C tokens at the last timed
step, one new token each, logits -> greedy token on the device -> ids read back (the reference's batched `tg`,
/root/reference/src/cli/main.cpp:1246-1254, reads each pass's results before the next).  Prints one JSON line:
`value` = decoded tokens a second at the default batch; `points` = the same at batch 1 and 64; `prefill` = one
2,048-token prompt from an empty cache; `roofline` = bytes the decode step has to read / its time against HBM's 8 TB/s;
`calibration` = what a device copy, a read-only pass and a square bf16 library product reach on this card.  The prefill
record's `frac` is its flops over the bf16 peak; beside it `hbm_frac` is the weights it has to read (the experts its
tokens picked, counted in the warm-up run) over its time against 8 TB/s: few rows an expert make the step a
weight-streaming one.
Token ids are a fixed LCG sequence; weights are N(0, 0.02) generated on the device.  The context before the timed
steps is built by running each request's prompt through the model (`context_fill` gives its rate).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4, help="untimed steps before the timed ones (at least 1)")
    ap.add_argument("--layers", type=int, default=0, help="layers to run (0: as many of the configuration's as fit)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=0, help="tokens each sequence holds at the last timed step (0: the configuration's)")
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-calibration", action="store_true", help="skip the copy, read and library-product rates of the card")
    ap.add_argument("--no-logits-to-host", action="store_true",
                    help="skip the extra point: the default batch with every step's logits copied to the host")
    ap.add_argument("--only-prefill", action="store_true", help="for profiling: measure the prefill alone and print its record")
    ap.add_argument("--context-fill", choices=["prefill", "synthetic"], default="prefill",
                    help="how the context before the timed steps gets into the cache: prompts run through the model in "
                         "portions of 2,048 tokens, or (for quick profiling runs) random keys and values written directly")
    return ap.parse_args()


# The real layer sizes: 24 layers of the 62-layer model's widths (the third configuration of the benchmark's list).
def real_config(layers: int, context: int):
    from llmx_amd import MiniMaxM3Config
    return MiniMaxM3Config(vocab_size=200064, hidden_size=3072, num_hidden_layers=layers, num_attention_heads=48,
                           num_key_value_heads=8, head_dim=128, rotary_dim=64, rope_theta=5e6, rms_norm_eps=1e-6,
                           num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536, routed_scaling_factor=1.0,
                           norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=max(context, PREFILL_TOKENS))


def lcg_ids(n, vocab, seed):
    x, out = (seed * 2654435761 + 1) & 0xFFFFFFFF, []
    for _ in range(n):
        x = (x * 1664525 + 1013904223) & 0xFFFFFFFF
        out.append((x >> 8) % vocab)
    return out


def layer_weight_bytes(c, wb):
    attn = (c.q_width + 2 * c.kv_width) * c.hidden_size * wb + c.hidden_size * c.q_width * wb
    router = c.num_local_experts * c.hidden_size * 4 + c.num_local_experts * 4
    norms = (2 * c.hidden_size + c.q_width + c.kv_width) * 4
    expert = 3 * c.intermediate_size * c.hidden_size * wb
    return attn, router + norms, expert


def decode_bytes(c, batch, context, distinct_experts, wb=2):
    """Bytes one decode step has to read: every weight it uses once, and the cache of the live requests."""
    attn, small, expert = layer_weight_bytes(c, wb)
    per_layer = attn + small + distinct_experts * expert
    head = c.vocab_size * c.hidden_size * wb + c.hidden_size * 4
    kv = batch * context * c.num_hidden_layers * 2 * c.kv_width * wb
    embed = batch * c.hidden_size * wb
    return c.num_hidden_layers * per_layer + head + kv + embed


def prefill_flops(c, T):
    per_layer = (2 * T * c.hidden_size * (c.q_width + 2 * c.kv_width) + 2 * T * c.q_width * c.hidden_size
                 + 4 * c.num_attention_heads * c.head_dim * T * (T + 1) // 2
                 + 2 * T * c.hidden_size * c.num_local_experts
                 + 2 * T * c.num_experts_per_tok * 3 * c.hidden_size * c.intermediate_size)
    return c.num_hidden_layers * per_layer + 2 * c.hidden_size * c.vocab_size


class DistinctExperts:
    """Observer: counts, per routed layer of a step, how many different experts the batch picked."""

    def __init__(self):
        self.counts = []

    def __call__(self, step, kind, **tensors):
        if kind == "routing":
            import torch
            self.counts.append(int(torch.unique(tensors["ids"]).numel()))


def calibrate(torch, device):
    """What this card gives a plain program: a device-to-device copy (bytes read plus written), a read-only pass
    (a kernel that streams 4 GiB and keeps nothing) and a square bf16 library product, beside the published 8 TB/s and 2.5 PFLOP/s."""
    def best(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        t = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            t.append(time.perf_counter() - t0)
        return min(t)
    n = 1 << 30
    src = torch.empty(n, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    copy_gbs = 2 * 4 * n / best(lambda: dst.copy_(src)) / 1e9
    from llmx_amd import ops
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    read_gbs = 4 * n / best(lambda: ops.read_probe(src, flag)) / 1e9
    del dst, src
    m = 8192
    a = torch.empty(m, m, dtype=torch.bfloat16, device=device).normal_()
    b = torch.empty(m, m, dtype=torch.bfloat16, device=device).normal_()
    tflops = 2 * m ** 3 / best(lambda: torch.matmul(a, b)) / 1e12
    del a, b
    torch.cuda.empty_cache()
    return {"copy_gbs": round(copy_gbs, 1), "read_gbs": round(read_gbs, 1), "bf16_gemm_tflops": round(tflops, 1)}


def run_decode(engine, sampler_out, batch, context, steps, warmup, fill, torch, read_logits=False):
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    c = engine.config
    start = context - (steps + warmup)
    if start < 1:
        raise SystemExit(f"bench: context {context} is shorter than the {steps + warmup} steps")
    rids = [f"b{batch}_{i}" for i in range(batch)]
    torch.cuda.synchronize()
    t_fill = time.perf_counter()
    for i, rid in enumerate(rids):
        engine.add_request(rid)
        if fill == "synthetic":
            engine.assume_context(rid, start)
        else:
            ids = lcg_ids(start, c.vocab_size, 100 + i)
            for s in range(0, start, PREFILL_TOKENS):
                engine.step([StepEntry(rid, ids[s:s + PREFILL_TOKENS], [])])
    torch.cuda.synchronize()
    run_decode.fill_s = time.perf_counter() - t_fill
    last = [lcg_ids(1, c.vocab_size, 7 + i)[0] for i in range(batch)]
    out = sampler_out[:batch]
    host_logits = torch.empty(batch, c.vocab_size, dtype=torch.float32, pin_memory=True) if read_logits else None

    def one():
        nonlocal last
        logits = engine.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, last)])
        ops.argmax_rows(logits, out)
        if read_logits:
            host_logits.copy_(logits)     # the reference's bench reads every step's logits on the host
        last = out.tolist()   # the ids come back to the host, as a serving loop reads them

    # the first warm-up step also counts the experts the batch touches per layer
    watcher = DistinctExperts()
    engine.observer = watcher
    one()
    engine.observer = None
    distinct = sum(watcher.counts) / max(1, len(watcher.counts))
    for _ in range(warmup - 1):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for rid in rids:
        engine.end_request(rid)
    return dt, distinct


def run_prefill(engine, cfg, sampler_out, torch):
    """One prompt of 2,048 tokens from an empty cache, in one step, to its first sampled token; best of two after a warm-up."""
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    T = PREFILL_TOKENS
    times = []
    watcher = DistinctExperts()
    for rep in range(3):   # the first is the warm-up; it also counts the experts the prompt touches per layer
        rid = f"p{rep}"
        engine.add_request(rid)
        ids = lcg_ids(T, cfg.vocab_size, 500 + rep)
        engine.observer = watcher if rep == 0 else None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry(rid, ids, [T - 1])])
        ops.argmax_rows(logits, sampler_out[:1])
        sampler_out[:1].tolist()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.end_request(rid)
    engine.observer = None
    t = min(times[1:])
    flops = prefill_flops(cfg, T)
    # what the step has to read: every weight it uses once (the experts the prompt's tokens picked), as for decode
    distinct = sum(watcher.counts) / max(1, len(watcher.counts))
    need = decode_bytes(cfg, 0, 0, distinct)
    return {"value": round(T / t, 1), "tokens": T, "ms": round(t * 1e3, 3), "frac": round(flops / t / PEAK_FLOPS["bf16"], 5),
            "tflop": round(flops / 1e12, 2), "distinct_experts_per_layer": round(distinct, 1), "weights_read_gb": round(need / 1e9, 1),
            "hbm_frac": round(need / t / 1e9 / HBM_PEAK_GBS, 4)}


def main():
    a = parse()
    a.warmup = max(1, a.warmup)
    if a.gpus != 1:
        print(f"bench: this engine runs on one GPU; --gpus {a.gpus} is not built")
        sys.exit(2)
    import torch
    from llmx_amd import Engine, RandomInit, ops
    from llmx_amd.engine import StepEntry

    full_layers, context = 24, 4096
    context = a.context or context
    layers = a.layers or full_layers
    points = [int(p) for p in a.points.split(",") if p.strip()]
    max_batch = max([a.batch] + points)
    cfg = real_config(layers, context)
    t_setup = time.perf_counter()
    engine = Engine.from_random(cfg, RandomInit(seed=0, std=0.02), dtype="bfloat16", kv_tokens=max_batch * context,
                                page_tokens=16, max_requests=max_batch)
    if a.context_fill == "synthetic":
        engine.fill_cache_random(seed=1)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup
    sampler_out = torch.empty(max_batch, dtype=torch.int32, device=engine.device)

    if a.only_prefill:
        print(json.dumps({"prefill": run_prefill(engine, cfg, sampler_out, torch)}))
        return
    dt, distinct = run_decode(engine, sampler_out, a.batch, context, a.steps, a.warmup, a.context_fill, torch)
    fill_s = run_decode.fill_s
    ms_per_step = dt / a.steps * 1e3
    value = a.batch * a.steps / dt
    mean_context = context - a.steps / 2
    need = decode_bytes(cfg, a.batch, mean_context, distinct)
    achieved = need / (dt / a.steps) / 1e9

    result = {
        "metric": "decode tok/s (MiniMax-M3 real layer sizes, batch %d, context %d)" % (a.batch, context),
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: LCG token ids, N(0,0.02) weights generated on the device; context before the timed steps: "
                + ("random keys and values written to the cache" if a.context_fill == "synthetic" else "prompts run through the model"),
        "config": {
            "model": "MiniMax-M3 slice (real layer sizes, configs[2])", "layers": layers, "layers_of_config": full_layers, "layers_full_model": 62,
            "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "rotary_dim": cfg.rotary_dim, "experts": cfg.num_local_experts, "top_k": cfg.num_experts_per_tok,
            "expert_intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "global_batch": a.batch, "seq_len": context,
            "page_tokens": 16, "parallelism": "single GPU", "weights_gb": round(engine.weight_bytes() / 1e9, 1),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_gb": round(need / 1e9, 2),
                     "distinct_experts_per_layer": round(distinct, 1)},
        "setup_s": round(setup_s, 1),
        **({"context_fill": {"tokens": a.batch * (context - a.steps - a.warmup), "s": round(fill_s, 2),
                             "tok_s": round(a.batch * (context - a.steps - a.warmup) / fill_s, 1), "portion": PREFILL_TOKENS}}
           if a.context_fill == "prefill" else {}),
    }

    pts = {}
    if points and not a.no_logits_to_host:
        dtb, _ = run_decode(engine, sampler_out, a.batch, context, a.steps, a.warmup, a.context_fill, torch, read_logits=True)
        pts[f"decode_b{a.batch}_logits_to_host"] = round(a.batch * a.steps / dtb, 2)
    for b in points:
        steps = a.steps
        dtb, _ = run_decode(engine, sampler_out, b, context, steps, a.warmup, a.context_fill, torch)
        pts[f"decode_b{b}"] = round(b * steps / dtb, 2)
    if pts:
        result["points"] = pts

    if not a.no_prefill:
        result["prefill"] = run_prefill(engine, cfg, sampler_out, torch)
    if not a.no_calibration:
        result["calibration"] = calibrate(torch, sampler_out.device)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
