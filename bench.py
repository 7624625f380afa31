"""Decode and prefill throughput of MiniMax-M3 at real layer sizes with random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C] [--points 1,64] [--no-sweep] [--no-long]

A step is one decode step of the whole batch: B requests, each at a context that reaches C tokens at the last timed
step, one new token each, logits -> greedy token on the device -> ids read back (the reference's batched `tg`,
/root/reference/src/cli/main.cpp:1246-1254, reads each pass's results before the next; it reports every test it times,
:1192-1287, and so does this line).  Prints one JSON line:
  value, ms_per_step   decoded tokens a second and the step's time at the default batch;
  roofline             bytes the decode step has to read (every weight it uses once, with the measured number of
                       distinct experts a layer, and the cache of the live requests) / its time, against HBM's 8 TB/s;
  points               the same for every measured batch, flat: decode_b<B> (tok/s), decode_b<B>_ms, _gb (bytes to read),
                       _experts (distinct a layer) and _frac (of 8 TB/s); decode_b<B>_logits_to_host is the default batch
                       with every step's logits copied to pinned host memory, as the reference's bench reads them;
                       generate_b<B>: the same batch through the product's own loop (scheduler, step, device sampler
                       with temperature 0.8, top-k 40, top-p 0.95): tok/s of its steps that carried only decoded
                       tokens, their mean rows (_rows_a_step) and time (_ms);
  prefill              one 2,048-token prompt from an empty cache: tok/s, ms, `frac` = flops / time / the bf16 peak,
                       `hbm_frac` = the weights it has to read (the experts its tokens picked) / time / 8 TB/s, and the
                       first layer's feed-forward alone (first_layer_*): its rows are all different, so it touches every
                       expert and streams all their weights;
  sweep                further sizes (left out with --no-sweep, or when --points is empty and --sweep is not given): batch 8
                       at 16k and 32k tokens of context, batch 16, 32 and 128 at 4k, batch 64 at 8k (tok/s, _ms, _frac;
                       batch 64 at 16k would hold 103 GB of cache beside 178.6 GB of weights and does not fit the card);
                       the mixed step a scheduler issues: a 512-token prompt portion beside 8 decoding requests;
                       generate_b1: batch 1 through the product's own loop with the default sampler, beside decode_b1;
                       prefill_8192: one prompt of 8,192 tokens in portions of 2,048 (tok/s, _ms, _frac of the bf16 peak);
                       prefill_spread: 2,048 rows as 64 requests of 32 tokens in one step, whose rows pick most experts in
                       every layer, so the step streams weights (_ms, _experts a layer, _frac of 8 TB/s);
  long                 the long-context configuration (left out with --no-long or when another --layers, --batch or
                       --context is asked for): 30 layers, 2 requests of 65,536 prompt tokens in portions of 2,048, then
                       256 decoded tokens each (the first engine is freed and another built for it);
  calibration          what a device copy, a read-only pass and a square bf16 library product reach on this card.
Token ids are a fixed LCG sequence; weights are N(0, 0.02) generated on the device.  The context before the timed steps
is built by running each request's prompt through the model in portions of 2,048 tokens (`context_fill` gives its rate).
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
FULL_LAYERS, CONTEXT = 24, 4096                     # the benchmark's configuration: 24 of the model's 62 layers, 4,096 tokens
LONG_LAYERS, LONG_PROMPT, LONG_DECODE = 30, 65536, 256


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4, help="untimed steps before the timed ones (at least 1)")
    ap.add_argument("--layers", type=int, default=0, help="layers to run (0: the configuration's 24)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=0, help="tokens each sequence holds at the last timed step (0: the configuration's 4,096)")
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--sweep", action="store_true", help="measure further contexts and batches and the mixed prompt + decode step (the default whenever --points names a batch)")
    ap.add_argument("--no-sweep", action="store_true", help="leave those out")
    ap.add_argument("--long", action="store_true", help="run the long-context configuration (30 layers, 2 x 65,536 tokens, 256 decoded) also beside a non-default run")
    ap.add_argument("--no-long", action="store_true", help="leave the long-context configuration out of the default run")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-calibration", action="store_true", help="skip the copy, read and library-product rates of the card")
    ap.add_argument("--no-logits-to-host", action="store_true",
                    help="skip the extra point: the default batch with every step's logits copied to the host")
    ap.add_argument("--no-generate", action="store_true", help="skip the extra point: the default batch through the scheduler and the sampler")
    ap.add_argument("--only-prefill", action="store_true", help="for profiling: measure the prefill alone and print its record")
    ap.add_argument("--only-long", action="store_true", help="for profiling: run the long-context configuration alone and print its record")
    return ap.parse_args()


def real_config(layers: int, positions: int):
    """The real layer sizes (the third configuration of the benchmark's list) with `layers` layers."""
    from llmx_amd import MiniMaxM3Config
    return MiniMaxM3Config(vocab_size=200064, hidden_size=3072, num_hidden_layers=layers, num_attention_heads=48,
                           num_key_value_heads=8, head_dim=128, rotary_dim=64, rope_theta=5e6, rms_norm_eps=1e-6,
                           num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536, routed_scaling_factor=1.0,
                           norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=max(positions, PREFILL_TOKENS))


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

    @property
    def mean(self):
        return sum(self.counts) / max(1, len(self.counts))


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


def fill_context(engine, rids, tokens_each, torch):
    """Runs each request's prompt of `tokens_each` tokens through the model in portions of 2,048; returns the seconds it took."""
    from llmx_amd.engine import StepEntry
    c = engine.config
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i, rid in enumerate(rids):
        engine.add_request(rid)
        ids = lcg_ids(tokens_each, c.vocab_size, 100 + i)
        for s in range(0, tokens_each, PREFILL_TOKENS):
            engine.step([StepEntry(rid, ids[s:s + PREFILL_TOKENS], [])])
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def run_decode(engine, sampler_out, batch, context, steps, warmup, torch, read_logits=False):
    """`steps` timed decode steps of `batch` requests that end at `context` tokens each.  Returns a record: seconds of the
    timed steps, of the context fill, and the distinct experts a layer that the first warm-up step touched."""
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    c = engine.config
    start = context - (steps + warmup)
    if start < 1:
        raise SystemExit(f"bench: context {context} is shorter than the {steps + warmup} steps")
    rids = [f"b{batch}_{i}" for i in range(batch)]
    fill_s = fill_context(engine, rids, start, torch)
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
    return {"s": dt, "fill_s": fill_s, "fill_tokens": batch * start, "distinct": watcher.mean}


def decode_record(cfg, batch, context, steps, run):
    """tok/s, ms a step, the bytes the step has to read and their share of the HBM peak."""
    step_s = run["s"] / steps
    need = decode_bytes(cfg, batch, context - steps / 2, run["distinct"])
    return {"tok_s": round(batch * steps / run["s"], 2), "ms": round(step_s * 1e3, 4), "gb": round(need / 1e9, 2),
            "experts": round(run["distinct"], 1), "gbs": round(need / step_s / 1e9, 1), "frac": round(need / step_s / 1e9 / HBM_PEAK_GBS, 4)}


def run_prefill(engine, cfg, sampler_out, torch):
    """One prompt of 2,048 tokens from an empty cache, in one step, to its first sampled token; best of two after a
    warm-up.  The first layer's feed-forward (router, routing, both routed products, combine) is timed by events of its own."""
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    T = PREFILL_TOKENS
    times, first_ms = [], []
    watcher = DistinctExperts()
    ffn = engine.model.blocks[0].ffn
    plain_forward = ffn.forward
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

    def timed_forward(*args, **kwargs):
        marks[0].record()
        plain_forward(*args, **kwargs)
        marks[1].record()

    ffn.forward = timed_forward
    try:
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
            first_ms.append(marks[0].elapsed_time(marks[1]))
            engine.end_request(rid)
    finally:
        ffn.forward = plain_forward
        engine.observer = None
    t = min(times[1:])
    flops = prefill_flops(cfg, T)
    # what the step has to read: every weight it uses once (the experts the prompt's tokens picked), as for decode
    need = decode_bytes(cfg, 0, 0, watcher.mean)
    first_experts = watcher.counts[0] if watcher.counts else 0
    _, small, expert = layer_weight_bytes(cfg, 2)
    first_bytes = first_experts * expert + small
    first = min(first_ms[1:]) * 1e-3
    return {"value": round(T / t, 1), "tokens": T, "ms": round(t * 1e3, 3), "frac": round(flops / t / PEAK_FLOPS["bf16"], 5),
            "tflop": round(flops / 1e12, 2), "distinct_experts_per_layer": round(watcher.mean, 1), "weights_read_gb": round(need / 1e9, 1),
            "hbm_frac": round(need / t / 1e9 / HBM_PEAK_GBS, 4),
            "first_layer_ffn_ms": round(first * 1e3, 3), "first_layer_experts": first_experts, "first_layer_gb": round(first_bytes / 1e9, 2),
            "first_layer_hbm_frac": round(first_bytes / first / 1e9 / HBM_PEAK_GBS, 4)}


def run_prefill_portions(engine, cfg, total, torch):
    """One prompt of `total` tokens from an empty cache in portions of 2,048 to its last row's logits; best of two."""
    from llmx_amd.engine import StepEntry
    times = []
    for rep in range(2):
        rid = f"pp{rep}"
        engine.add_request(rid)
        ids = lcg_ids(total, cfg.vocab_size, 600 + rep)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(0, total, PREFILL_TOKENS):
            part = ids[s:s + PREFILL_TOKENS]
            engine.step([StepEntry(rid, part, [len(part) - 1] if s + len(part) == total else [])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.end_request(rid)
    t = min(times)
    return {"tok_s": round(total / t, 1), "ms": round(t * 1e3, 3), "frac": round(prefill_flops(cfg, total) / t / PEAK_FLOPS["bf16"], 4)}


def run_prefill_spread(engine, cfg, requests, tokens_each, torch):
    """`requests` prompts of `tokens_each` tokens in one step from an empty cache.  Short prompts of different tokens keep
    their rows apart through the layers, so every layer's rows pick most of the experts: the step has to stream their
    weights, where one long prompt's rows (which grow alike with random weights) pick few.  Best of two after a warm-up."""
    from llmx_amd.engine import StepEntry
    watcher = DistinctExperts()
    times = []
    for rep in range(3):
        rids = [f"ps{rep}_{i}" for i in range(requests)]
        entries = []
        for i, rid in enumerate(rids):
            engine.add_request(rid)
            entries.append(StepEntry(rid, lcg_ids(tokens_each, cfg.vocab_size, 3000 + 97 * rep + i), [tokens_each - 1]))
        engine.observer = watcher if rep == 0 else None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step(entries)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.observer = None
        for rid in rids:
            engine.end_request(rid)
    t = min(times[1:])
    need = decode_bytes(cfg, 0, 0, watcher.mean)
    return {"ms": round(t * 1e3, 3), "experts": round(watcher.mean, 1), "gb": round(need / 1e9, 1), "frac": round(need / t / 1e9 / HBM_PEAK_GBS, 4),
            "tok_s": round(requests * tokens_each / t, 1)}


def run_mixed_step(engine, cfg, sampler_out, context, portion, decoding, reps, torch):
    """The step a scheduler issues while a prompt arrives: `decoding` requests at `context` tokens take one token each
    beside a `portion`-token portion of another request's prompt.  Returns ms a step (mean of `reps`) and tokens a second."""
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    rids = [f"m{i}" for i in range(decoding)]
    fill_context(engine, rids, context - reps - 1, torch)
    engine.add_request("prompt")
    ids = lcg_ids(portion * (reps + 1), cfg.vocab_size, 900)
    last = [lcg_ids(1, cfg.vocab_size, 7 + i)[0] for i in range(decoding)]
    out = sampler_out[:decoding]

    def one(k):
        nonlocal last
        entries = [StepEntry(rid, [t], [0]) for rid, t in zip(rids, last)] + [StepEntry("prompt", ids[k * portion:(k + 1) * portion], [])]
        ops.argmax_rows(engine.step(entries), out)
        last = out.tolist()

    one(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(1, reps + 1):
        one(k)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    for rid in rids + ["prompt"]:
        engine.end_request(rid)
    return {"ms": round(dt * 1e3, 3), "tok_s": round((decoding + portion) / dt, 1), "decoding": decoding, "portion": portion, "context": context}


def run_generate(engine, cfg, batch, context, new_tokens, torch):
    """The product's own loop: `batch` requests through the scheduler (prompts in portions beside decoding requests),
    the step function and the device sampler with the reference's default settings (temperature 0.8, top-k 40, top-p
    0.95), each request's context reaching `context` tokens.  Reports the steps that carried only decoded tokens."""
    from llmx_amd import SamplingParams
    from llmx_amd.engine.generation import Generator
    from llmx_amd.engine.scheduler import Request
    gen = Generator(engine, batch, PREFILL_TOKENS)
    for i in range(batch):
        gen.submit(Request(("generate", i), lcg_ids(context - new_tokens, cfg.vocab_size, 100 + i),
                           SamplingParams(max_tokens=new_tokens, temp=0.8, top_k=40, top_p=0.95, seed=1 + i, ignore_eos=True)))
    gen.run()
    torch.cuda.synchronize()
    st = gen.stats
    return {"tok_s": round(st.decode_rows / max(st.decode_seconds, 1e-9), 2), "rows_a_step": round(st.decode_rows / max(st.decode_steps, 1), 2),
            "ms": round(st.decode_seconds / max(st.decode_steps, 1) * 1e3, 4)}


def run_long(torch, steps_warm=4):
    """The long-context configuration: 30 layers, 2 requests of 65,536 prompt tokens fed in portions of 2,048, then 256
    decoded tokens each.  Returns its record."""
    from llmx_amd import Engine, RandomInit, ops
    from llmx_amd.engine import StepEntry
    batch, context = 2, LONG_PROMPT + LONG_DECODE
    cfg = real_config(LONG_LAYERS, context)
    engine = Engine.from_random(cfg, RandomInit(seed=0, std=0.02), dtype="bfloat16", kv_tokens=batch * context, page_tokens=16, max_requests=batch)
    rids = [f"long{i}" for i in range(batch)]
    fill_s = fill_context(engine, rids, LONG_PROMPT, torch)
    out = torch.empty(batch, dtype=torch.int32, device=engine.device)
    last = [lcg_ids(1, cfg.vocab_size, 7 + i)[0] for i in range(batch)]
    watcher = DistinctExperts()

    def one():
        nonlocal last
        ops.argmax_rows(engine.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, last)]), out)
        last = out.tolist()

    engine.observer = watcher
    one()
    engine.observer = None
    for _ in range(steps_warm - 1):
        one()
    torch.cuda.synchronize()
    timed = LONG_DECODE - steps_warm
    t0 = time.perf_counter()
    for _ in range(timed):
        one()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    record = decode_record(cfg, batch, context, timed, {"s": dt, "distinct": watcher.mean})
    for rid in rids:
        engine.end_request(rid)
    weights_gb = engine.weight_bytes() / 1e9
    del engine
    torch.cuda.empty_cache()
    return {"layers": LONG_LAYERS, "batch": batch, "prompt_tokens": LONG_PROMPT, "portion": PREFILL_TOKENS, "decoded": LONG_DECODE,
            "weights_gb": round(weights_gb, 1), "prompt_s": round(fill_s, 2), "prompt_tok_s": round(batch * LONG_PROMPT / fill_s, 1),
            "decode_tok_s": record["tok_s"], "decode_ms": record["ms"], "decode_gb": record["gb"], "decode_frac": record["frac"]}


def main():
    a = parse()
    a.warmup = max(1, a.warmup)
    if a.gpus != 1:
        print(f"bench: this engine runs on one GPU; --gpus {a.gpus} is not built")
        sys.exit(2)
    import torch
    from llmx_amd import Engine, RandomInit

    if a.only_long:
        print(json.dumps({"long": run_long(torch)}))
        return
    context = a.context or CONTEXT
    layers = a.layers or FULL_LAYERS
    points = [int(p) for p in a.points.split(",") if p.strip()]
    do_sweep = a.sweep or (bool(points) and not a.no_sweep)
    # the long-context configuration belongs to the default run; a run at other sizes (a test, a profile) asks for it
    do_long = a.long or (not a.no_long and not (a.layers or a.context) and a.batch == 8 and bool(points))
    sweep = [(8, 16384), (8, 32768), (16, context), (32, context), (128, context), (64, 2 * context)] if do_sweep else []
    kv_tokens = max([a.batch * context] + [b * context for b in points] + [b * c for b, c in sweep] + ([9 * context] if do_sweep else []))
    max_batch = max([a.batch] + points + [b for b, _ in sweep] + ([64] if do_sweep else []))
    cfg = real_config(layers, max([context] + [c for _, c in sweep]))
    t_setup = time.perf_counter()
    engine = Engine.from_random(cfg, RandomInit(seed=0, std=0.02), dtype="bfloat16", kv_tokens=kv_tokens, page_tokens=16, max_requests=max_batch)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup
    sampler_out = torch.empty(max_batch, dtype=torch.int32, device=engine.device)

    if a.only_prefill:
        print(json.dumps({"prefill": run_prefill(engine, cfg, sampler_out, torch)}))
        return
    run = run_decode(engine, sampler_out, a.batch, context, a.steps, a.warmup, torch)
    head = decode_record(cfg, a.batch, context, a.steps, run)

    result = {
        "metric": "decode tok/s (MiniMax-M3 real layer sizes, batch %d, context %d)" % (a.batch, context),
        "value": head["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: LCG token ids, N(0,0.02) weights generated on the device; context before the timed steps: prompts run through the model",
        "config": {
            "model": "MiniMax-M3 slice (real layer sizes, configs[2])", "layers": layers, "layers_of_config": FULL_LAYERS, "layers_full_model": 62,
            "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "rotary_dim": cfg.rotary_dim, "experts": cfg.num_local_experts, "top_k": cfg.num_experts_per_tok,
            "expert_intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "global_batch": a.batch, "seq_len": context,
            "page_tokens": 16, "parallelism": "single GPU", "weights_gb": round(engine.weight_bytes() / 1e9, 1),
        },
        "roofline": {"bound": "hbm", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac"],
                     "bytes_gb": head["gb"], "distinct_experts_per_layer": head["experts"]},
        "setup_s": round(setup_s, 1),
        "context_fill": {"tokens": run["fill_tokens"], "s": round(run["fill_s"], 2), "tok_s": round(run["fill_tokens"] / run["fill_s"], 1),
                         "portion": PREFILL_TOKENS},
    }

    pts = {}

    def add_point(name, rec):
        pts[name] = rec["tok_s"]
        for key in ("ms", "gb", "experts", "frac"):
            pts[f"{name}_{key}"] = rec[key]

    add_point(f"decode_b{a.batch}", head)
    if points and not a.no_logits_to_host:
        r = run_decode(engine, sampler_out, a.batch, context, a.steps, a.warmup, torch, read_logits=True)
        pts[f"decode_b{a.batch}_logits_to_host"] = round(a.batch * a.steps / r["s"], 2)
    for b in points:
        add_point(f"decode_b{b}", decode_record(cfg, b, context, a.steps, run_decode(engine, sampler_out, b, context, a.steps, a.warmup, torch)))
    if points and not a.no_generate:
        g = run_generate(engine, cfg, a.batch, context, 2 * a.steps, torch)
        for key, v in g.items():
            pts[f"generate_b{a.batch}" if key == "tok_s" else f"generate_b{a.batch}_{key}"] = v
    result["points"] = pts

    if do_sweep:
        sw = {}
        for b, c in sweep:
            rec = decode_record(cfg, b, c, a.steps, run_decode(engine, sampler_out, b, c, a.steps, a.warmup, torch))
            name = f"decode_b{b}_ctx{c}"
            sw[name] = rec["tok_s"]
            for key in ("ms", "frac"):
                sw[f"{name}_{key}"] = rec[key]
        mixed = run_mixed_step(engine, cfg, sampler_out, context, 512, 8, 8, torch)
        sw["mixed_512_beside_8_ms"] = mixed["ms"]
        sw["mixed_512_beside_8_tok_s"] = mixed["tok_s"]
        # batch 1 through the scheduler, the step and the device sampler, beside the bare step of decode_b1
        g1 = run_generate(engine, cfg, 1, context, 2 * a.steps, torch)
        sw["generate_b1"], sw["generate_b1_ms"] = g1["tok_s"], g1["ms"]
        if "decode_b1_gb" in pts:
            sw["generate_b1_frac"] = round(pts["decode_b1_gb"] / g1["ms"] / (HBM_PEAK_GBS / 1e3), 4)
        if not a.no_prefill:
            p8 = run_prefill_portions(engine, cfg, 4 * PREFILL_TOKENS, torch)
            sw["prefill_8192"], sw["prefill_8192_ms"], sw["prefill_8192_frac"] = p8["tok_s"], p8["ms"], p8["frac"]
            sp = run_prefill_spread(engine, cfg, 64, PREFILL_TOKENS // 64, torch)
            sw["prefill_spread_ms"], sw["prefill_spread_experts"], sw["prefill_spread_frac"] = sp["ms"], sp["experts"], sp["frac"]
        result["sweep"] = sw

    if not a.no_prefill:
        result["prefill"] = run_prefill(engine, cfg, sampler_out, torch)
    if not a.no_calibration:
        result["calibration"] = calibrate(torch, sampler_out.device)
    if do_long:
        del engine
        torch.cuda.empty_cache()
        result["long"] = run_long(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
