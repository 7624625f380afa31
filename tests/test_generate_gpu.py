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
