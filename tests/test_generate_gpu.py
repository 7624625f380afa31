"""Generation through the entry point: greedy against the plain implementation, seeded temperature sampling equal to
each request's run alone, the command line."""

from __future__ import annotations

import os
import subprocess
import sys

import pytest
import torch

import plain_model
from helpers import TINY, model_folder, plain, tokens_for

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine_for(name, dtype="float32", kv_tokens=512, max_requests=4, page=None):
    from llmx_amd import Engine
    return Engine.load(model_folder(name), dtype=dtype, kv_tokens=kv_tokens, page_tokens=page or TINY[name][2], max_requests=max_requests)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_equals_the_plain_implementation(name):
    """Three prompts (lengths 5, 17, 32 for A; 1, 9, 23, 40 for B), 8 greedy tokens each, generated together."""
    from llmx_amd import SamplingParams, generate
    cfg, w = plain(name)
    lengths = (5, 17, 32) if name == "A" else (1, 9, 23, 40)
    prompts = [tokens_for(name, n, 40 + i) for i, n in enumerate(lengths)]
    want = [plain_model.greedy(cfg, w, p, 8) for p in prompts]
    engine = engine_for(name, "float32")
    got = generate(engine, prompts, SamplingParams(max_tokens=8, temp=0.0), max_step_tokens=7)
    assert got == want
    assert engine.cache.pages_in_use() == 0
    # and alone, in one step per prompt
    for p, wnt in zip(prompts, want):
        assert generate(engine, [p], SamplingParams(max_tokens=8, temp=0.0))[0] == wnt
    # bfloat16 generates valid tokens of the right count (its picks may differ where two logits are close)
    got16 = generate(engine_for(name, "bfloat16"), prompts, SamplingParams(max_tokens=8, temp=0.0), max_step_tokens=7)
    assert [len(g) for g in got16] == [8] * len(prompts)
    agree = sum(a == b for g, wnt in zip(got16, want) for a, b in zip(g[:1], wnt[:1]))
    assert agree >= len(prompts) - 1


def test_seeded_temperature_sampling_is_each_request_alone():
    """Configuration B's run: prompts of 1, 9, 23 and 40 tokens prefilled in 7-token portions mixed with decode steps,
    temperature 0.8 with a fixed seed.  Every request owns its generator, so its tokens equal its run alone."""
    from llmx_amd import SamplingParams, generate
    name = "B"
    prompts = [tokens_for(name, n, 60 + i) for i, n in enumerate((1, 9, 23, 40))]
    params = [SamplingParams(max_tokens=12, temp=0.8, top_k=0, top_p=1.0, seed=1234 + i) for i in range(4)]
    engine = engine_for(name, "float32")
    together = generate(engine, prompts, params, max_seqs=3, max_step_tokens=7)
    alone = [generate(engine, [p], sp)[0] for p, sp in zip(prompts, params)]
    assert together == alone
    again = generate(engine, prompts, params, max_seqs=4, max_step_tokens=512)
    assert again == together
    other_seed = generate(engine, prompts[3:], SamplingParams(max_tokens=12, temp=0.8, top_k=0, top_p=1.0, seed=99))[0]
    assert other_seed != together[3]
    # the default settings (top-k 40, top-p 0.95) run too, and penalties
    out = generate(engine, prompts, SamplingParams(max_tokens=6, seed=5, penalty=1.3, presence_penalty=0.2, frequency_penalty=0.1))
    assert all(len(o) == 6 for o in out)


def test_eos_ends_a_request():
    from llmx_amd import Engine, SamplingParams, generate
    name = "A"
    cfg, w = plain(name)
    prompt = tokens_for(name, 9, 77)
    free = plain_model.greedy(cfg, w, prompt, 6)
    engine = engine_for(name)
    engine.spec.eos_token_id = free[3]                    # the fourth greedy token becomes the end token
    assert generate(engine, [prompt], SamplingParams(max_tokens=6, temp=0.0))[0] == free[:3]
    ignoring = generate(engine, [prompt], SamplingParams(max_tokens=6, temp=0.0, ignore_eos=True))[0]
    assert len(ignoring) == 6 and ignoring[:3] == free[:3] and free[3] not in ignoring[3:4]


def test_a_stop_sequence_ends_a_request():
    from llmx_amd import Engine, SamplingParams, generate
    name = "B"
    cfg, w = plain(name)
    prompt = tokens_for(name, 9, 31)
    free = plain_model.greedy(cfg, w, prompt, 8)
    engine = engine_for(name)
    got = generate(engine, [prompt, prompt], [SamplingParams(max_tokens=8, temp=0.0, stop=tuple(free[3:5])),
                                              SamplingParams(max_tokens=8, temp=0.0, stop=((free[1], free[0]),))])
    at = next(i for i in range(1, 8) if free[i - 1:i + 1] == free[3:5])      # the pair's first appearance
    assert got[0] == free[:at + 1]                                            # the completing token is kept
    pairs = [free[i - 1:i + 1] for i in range(1, 8)]
    if [free[1], free[0]] not in pairs:
        assert got[1] == free                                                 # a sequence that never appears stops nothing


def test_wrappers_over_step_and_perplexity():
    """prefill, decode_one and score are the step function for one request; perplexity in windows, through the prompt
    path and token by token, equals the plain implementation's log-softmax in double."""
    from llmx_amd.engine.perplexity import perplexity
    name = "A"
    cfg, w = plain(name)
    ids = tokens_for(name, 45, 13)
    logits = plain_model.forward(cfg, w, ids).double()
    engine = engine_for(name)
    engine.add_request("r")
    row = engine.prefill("r", ids[:30], portion=7)
    assert (row.cpu() - logits[29].float()).abs().max() < 2e-5
    row = engine.decode_one("r", ids[30])
    assert (row.cpu() - logits[30].float()).abs().max() < 2e-5 and engine.length("r") == 31
    engine.end_request("r")
    engine.add_request("s")
    rows = engine.score("s", ids, portion=11)
    engine.end_request("s")
    assert rows.shape == (45, cfg["vocab_size"]) and (rows.cpu() - logits.float()).abs().max() < 2e-5

    def plain_nll(window):
        z = plain_model.forward(cfg, w, window).double()
        lp = torch.log_softmax(z, dim=1)
        return -sum(float(lp[i, window[i + 1]]) for i in range(len(window) - 1))
    want = [plain_nll(ids[0:20]), plain_nll(ids[20:40]), plain_nll(ids[40:45])]
    for per_token in (False, True):
        r = perplexity(engine, ids, context=20, per_token=per_token, portion=6)
        assert [s for s, _ in r.windows] == [19, 19, 4] and r.used_tokens == 45 and r.scored_tokens == 42
        for (scored, got), w_ in zip(r.windows, want):
            assert abs(got - w_) < 4e-5 * scored          # a logit and the log of the sum within 2e-5 each
        assert abs(r.mean_nll - sum(want) / 42) < 2e-5
    two = perplexity(engine, ids, context=20, max_chunks=2)
    assert len(two.windows) == 2 and two.scored_tokens == 38
    assert perplexity(engine, ids[:41], context=20).used_tokens == 40       # a rest of one token scores nothing
    with pytest.raises(ValueError, match="at least 2"):
        perplexity(engine, ids[:1])
    assert all(engine.cache.pages_in_use(g) == 0 for g in range(len(engine.cache.groups)))


def test_command_line(tmp_path):
    name = "A"
    cfg, w = plain(name)
    prompt = tokens_for(name, 11, 5)
    want = plain_model.greedy(cfg, w, prompt, 5)
    cmd = [os.path.join(ROOT, "bin", "llmx"), "generate", model_folder(name), ",".join(map(str, prompt)), "-n", "5", "--temp", "0",
           "--dtype", "f32", "--page-tokens", "4", "--verbose"]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.strip().split("\n")[-1].split() == [str(t) for t in want]
    assert "pp: 11 tok" in run.stderr and "tg: 5 tok" in run.stderr and "ids: " + ",".join(map(str, want)) in run.stderr
    bad = subprocess.run(cmd + ["--temp", "1"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2 and "given twice" in bad.stderr
    bad = subprocess.run(cmd[:4] + ["--no-such-flag"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2
    lg = subprocess.run([os.path.join(ROOT, "bin", "llmx"), "logits", model_folder(name), ",".join(map(str, prompt)), "--last", "2", "--top", "3",
                         "--dtype", "f32", "--page-tokens", "4"], capture_output=True, text=True, timeout=300)
    assert lg.returncode == 0, lg.stderr[-2000:]
    lines = lg.stdout.strip().split("\n")
    assert lines[0] == "tokens: 11" and len(lines) == 3
    logits = plain_model.forward(cfg, w, prompt)
    last = lines[-1].split()
    assert int(last[0]) == 10 and int(last[1]) == int(logits[-1].argmax()) and abs(float(last[2]) - float(logits[-1].max())) < 1e-4
    # --then-ids appends ids from a file; without --last the top list of the last position comes one id a line
    more = tmp_path / "more.txt"
    more.write_text(" ".join(map(str, prompt[6:])))
    lg = subprocess.run([os.path.join(ROOT, "bin", "llmx"), "logits", model_folder(name), ",".join(map(str, prompt[:6])), "--then-ids", str(more),
                         "--top", "3", "--dtype", "f32", "--page-tokens", "4", "--per-token"], capture_output=True, text=True, timeout=300)
    assert lg.returncode == 0, lg.stderr[-2000:]
    lines = lg.stdout.strip().split("\n")
    assert lines[0] == "tokens: 11" and len(lines) == 4 and int(lines[1].split()[0]) == int(logits[-1].argmax())
    ids_file = tmp_path / "ids.txt"
    ids_file.write_text(",".join(map(str, prompt * 3)))
    pp = subprocess.run([os.path.join(ROOT, "bin", "llmx"), "perplexity", model_folder(name), "--file", str(ids_file), "-c", "16", "--chunks", "2",
                         "--dtype", "f32", "--page-tokens", "4", "--verbose"], capture_output=True, text=True, timeout=300)
    assert pp.returncode == 0, pp.stderr[-2000:]
    out = dict(line.split(": ", 1) for line in pp.stdout.strip().split("\n") if not line.startswith("chunk "))
    assert out["tokens"] == "33" and out["used tokens"] == "32" and out["scored tokens"] == "30" and out["chunks"] == "2" and out["context size"] == "16"
    z = [torch.log_softmax(plain_model.forward(cfg, w, (prompt * 3)[s:s + 16]).double(), dim=1) for s in (0, 16)]
    nll = -sum(float(z[k][i, (prompt * 3)[16 * k + i + 1]]) for k in range(2) for i in range(15)) / 30
    assert abs(float(out["mean NLL"]) - nll) < 2e-5
    bad = subprocess.run([os.path.join(ROOT, "bin", "llmx"), "perplexity", model_folder(name), "7"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2 and "at least 2" in bad.stderr


def test_command_line_runs_a_configuration_with_random_weights(tmp_path):
    """`llmx generate --config JSON --random SEED`: weights come from the seed on the device, no folder is read or
    written; the tokens are those of an engine made from the same configuration and seed in this process."""
    import json
    from helpers import TINY_B
    from llmx_amd import Engine, MiniMaxM3Config, RandomInit, SamplingParams, generate
    cfg = MiniMaxM3Config(**TINY_B)
    path = tmp_path / "config.json"
    path.write_text(json.dumps(cfg.to_json()))
    prompt = tokens_for("B", 9, 3)
    engine = Engine.from_random(cfg, RandomInit(seed=5, std=0.05), dtype="float32", kv_tokens=64, page_tokens=8, max_requests=1)
    want = generate(engine, [prompt], SamplingParams(max_tokens=6, temp=0.0))[0]
    cmd = [os.path.join(ROOT, "bin", "llmx"), "generate", "--config", str(path), "--random", "5", "--std", "0.05", ",".join(map(str, prompt)),
           "-n", "6", "--temp", "0", "--dtype", "f32", "--page-tokens", "8"]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.strip().split("\n")[-1].split() == [str(t) for t in want]
    lg = subprocess.run([os.path.join(ROOT, "bin", "llmx"), "logits", "--config", str(path), "--random", "5", "--std", "0.05",
                         ",".join(map(str, prompt)), "--top", "1", "--dtype", "f32", "--page-tokens", "8"], capture_output=True, text=True, timeout=300)
    assert lg.returncode == 0, lg.stderr[-2000:]
    assert int(lg.stdout.strip().split("\n")[-1].split()[0]) == want[0]


def test_command_line_bench_of_a_model(tmp_path):
    """`llmx bench --model DIR --p --n --r --seqs --depth` prints the reference's lines (`bench: pp16 ...`,
    `bench: tg8 ...`, `bench: x3 tg8 ...`, ` @ d40` after a history; /root/reference/src/cli/main.cpp:1261-1270) and
    leaves no request open between its runs (every run opens its requests anew in a pool made for one run)."""
    import re
    exe = os.path.join(ROOT, "bin", "llmx")
    one = subprocess.run([exe, "bench", "--model", model_folder("A16"), "--p", "16", "--n", "8", "--r", "2", "--depth", "40", "--ubatch", "12"],
                         capture_output=True, text=True, timeout=300)
    assert one.returncode == 0, one.stderr[-2000:]
    lines = [l for l in one.stdout.strip().split("\n") if l.startswith("bench: ")]
    assert len(lines) == 2
    assert re.fullmatch(r"bench: pp16 @ d40 +[0-9.]+ \+- [0-9.]+ tok/s  \(2 runs\)", lines[0]), lines[0]
    assert re.fullmatch(r"bench: tg8 @ d40 +[0-9.]+ \+- [0-9.]+ tok/s  \(2 runs\)", lines[1]), lines[1]
    import json
    from helpers import TINY_B
    from llmx_amd import MiniMaxM3Config
    path = tmp_path / "config.json"
    path.write_text(json.dumps(MiniMaxM3Config(**TINY_B).to_json()))
    many = subprocess.run([exe, "bench", "--config", str(path), "--random", "1", "--p", "9", "--n", "5", "--r", "1", "--seqs", "3", "--dtype", "f32",
                           "--page-tokens", "8"], capture_output=True, text=True, timeout=300)
    assert many.returncode == 0, many.stderr[-2000:]
    lines = [l for l in many.stdout.strip().split("\n") if l.startswith("bench: ")]
    assert lines[0].startswith("bench: pp9 ") and lines[1].startswith("bench: x3 tg5 ") and lines[1].endswith("(1 runs)")
    bad = subprocess.run([exe, "bench", "--model", model_folder("A16"), "--seqs", "2", "--depth", "5"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2 and "--depth" in bad.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_through_a_small_pool_equal_their_runs_alone(dtype):
    """Thirty requests of drawn lengths, counts and settings, through pages for about three of them: requests wait for
    pages, portions of prompts run beside decoded tokens, freed pages are used again.  Logits do not depend on the
    batch or the pages and every request owns its generator, so each gets the tokens of its run alone, bit for bit,
    in both dtypes."""
    import random
    from llmx_amd import SamplingParams, generate
    name = "B"
    rng = random.Random(5)
    prompts = [tokens_for(name, rng.randrange(1, 90), 200 + i) for i in range(30)]
    params = []
    for i in range(30):
        kind = i % 3
        params.append(SamplingParams(max_tokens=rng.randrange(1, 20), seed=77 + i, temp=(0.0, 0.8, 1.2)[kind],
                                     top_k=(0, 0, 12)[kind], top_p=(1.0, 1.0, 0.9)[kind],
                                     penalty=1.2 if i % 5 == 0 else 1.0, ignore_eos=True))
    small = engine_for(name, dtype, kv_tokens=3 * 112, max_requests=4)
    together = generate(small, prompts, params, max_seqs=4, max_step_tokens=48)
    assert small.cache.pages_in_use() == 0
    assert [len(t) for t in together] == [p.max_tokens for p in params]
    roomy = engine_for(name, dtype, kv_tokens=512, max_requests=2)
    for i, (prompt, sp) in enumerate(zip(prompts, params)):
        assert generate(roomy, [prompt], sp)[0] == together[i], f"request {i} ({len(prompt)} prompt tokens, {sp})"
