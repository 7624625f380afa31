"""bin/trace_run driven as a user drives it: a subprocess, steps on standard input, logits files out.

The same requests are replayed whole, with the last 32 tokens one by one, in portions of changing size, and mixed with
other requests in a pool so small that pages are used again; float32 and bfloat16; all compared with the plain
implementation, and with each other bit for bit."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import TINY, model_folder, plain_logits, plain_logits_with_picks, portions, tokens_for

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def replay(name, dtype, steps, out_dir, max_tokens, extra=()):
    """Runs trace_run over `steps`; returns {step: logits array [wanted, vocab]}; checks the `done` lines."""
    vocab = TINY[name][0]["vocab_size"]
    cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(name), "--dtype", dtype, "--out", str(out_dir),
           "--max-tokens", str(max_tokens), *extra]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    run = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.split("\n")[:len(steps)] == [f"done {s['step']}" for s in steps]
    out = {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = out_dir / f"{s['step']}.f32"
        if wanted:
            out[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not path.exists()
    return out


def whole_steps(requests):
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def cut_steps(rid, toks, cuts, first_step=0):
    steps = [{"step": first_step + i, "entries": [{"id": rid, "tokens": toks[a:b], "want": list(range(b - a))}], "end": []}
             for i, (a, b) in enumerate(cuts)]
    steps[-1]["end"] = [rid]
    return steps


def mixed_steps(requests, live_max=4):
    """Portions of some requests beside decoded tokens of others; requests start and end at different steps."""
    ids = list(requests)
    at = {r: 0 for r in ids}
    waiting, live, steps = list(ids), [], []
    where = {r: [] for r in ids}   # request -> [(step, first row, n)]
    step_no = 0
    while waiting or live:
        while waiting and len(live) < live_max:
            live.append(waiting.pop(0))
        entries, row = [], 0
        for slot, r in enumerate(live):
            total = len(requests[r])
            decode_from = max(1, total - 8)
            n = 1 if at[r] >= decode_from else min((5, 2, 11, 3, 7)[(step_no + slot) % 5], decode_from - at[r])
            if (step_no + slot) % 6 == 5 and len(live) > 1:
                continue
            entries.append({"id": r, "tokens": requests[r][at[r]:at[r] + n], "want": list(range(n))})
            where[r].append((step_no, row, n))
            row += n
            at[r] += n
        ended = [r for r in live if at[r] == len(requests[r])]
        live = [r for r in live if r not in ended]
        steps.append({"step": step_no, "entries": entries, "end": ended})
        step_no += 1
    return steps, where


LENGTHS = {"A": [75, 40, 23, 67, 9, 52], "B": [67, 40, 23, 9, 1, 52]}


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16")])
def test_replay_every_cutting(name, dtype, tmp_path):
    page = TINY[name][2]
    requests = {f"r{i}": tokens_for(name, n, 20 + i) for i, n in enumerate(LENGTHS[name])}
    tol = 2e-5 if dtype == "float32" else 2e-2
    extra = ["--page-tokens", str(page)]

    cfg = TINY[name][0]
    n_layers, k, X = cfg["num_hidden_layers"], cfg["num_experts_per_tok"], cfg["num_local_experts"]

    def check(rid, got, step_dir=None, step_no=None):
        """Every row against the plain implementation.  In bfloat16 a router key within rounding of a tie may fall either
        way, so the plain implementation runs with the picks the replay wrote (--routing), each checked against the
        replay's own router logits."""
        n = len(requests[rid])
        if dtype == "bfloat16":
            picks = torch.from_numpy(np.fromfile(step_dir / f"{step_no}.picks.i32", dtype="<i4").reshape(n_layers, n, k).astype(np.int64))
            router = torch.from_numpy(np.fromfile(step_dir / f"{step_no}.router.f32", dtype="<f4").reshape(n_layers, n, X))
            want = plain_logits_with_picks(name, requests[rid], list(picks), engine_logits=list(router)).numpy()
        else:
            want = plain_logits(name, n, 20 + int(rid[1:]), False).numpy()
        err = np.abs(got.astype(np.float64) - want).max()
        assert err <= tol * np.abs(want).max(), f"{rid}: max error {err:.3e}"

    # 1. each request alone and whole: compared with the plain implementation; the other cuttings must equal these bit for bit
    whole = replay(name, dtype, whole_steps(requests), tmp_path / "whole", max_tokens=128, extra=extra + ["--routing"])
    golden = {rid: whole[i] for i, rid in enumerate(requests)}
    for i, (rid, got) in enumerate(golden.items()):
        assert np.isfinite(got).all()
        check(rid, got, tmp_path / "whole", i)
    # 2. most in one step, the last 32 tokens one by one;  3. portions of changing size, down to two tokens
    rid = "r0"
    toks = requests[rid]
    n = len(toks)
    for label, cuts in (("last32", [(0, n - 32)] + [(i, i + 1) for i in range(n - 32, n)]), ("portions", portions(n))):
        out = replay(name, dtype, cut_steps(rid, toks, cuts), tmp_path / label, max_tokens=128, extra=extra)
        got = np.concatenate([out[i] for i in range(len(cuts))])
        assert np.array_equal(got, golden[rid]), f"{label}: differs from the whole prompt in {dtype}"
    # 4. mixed, up to four live requests, in a pool of four requests' worth of pages
    steps, where = mixed_steps(requests)
    # the pool: the most tokens live requests hold at any time, each request's count rounded up to a multiple of 64
    held, live_need = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        live_need = max(live_need, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in st["end"]:
            del held[rid]
    assert live_need < sum(-(-x // 64) * 64 for x in LENGTHS[name]), "the pool holds every request at once: no page is used again"
    out = replay(name, dtype, steps, tmp_path / "mixed", max_tokens=live_need, extra=extra)
    for rid in requests:
        got = np.concatenate([out[s][row:row + n_rows] for s, row, n_rows in where[rid]])
        assert np.array_equal(got, golden[rid]), f"{rid} in the mix differs from its run alone in {dtype}"


def test_replay_default_page_and_empty_want(tmp_path):
    """Default page size (16 tokens: the matrix-core attention path in bfloat16), steps that want nothing, a request
    left out of steps, ids reused after their end."""
    name = "A"
    toks = tokens_for(name, 50, 3)
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": toks[:20], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "y", "tokens": toks[:7], "want": [6]}], "end": ["y"]},
        {"step": 2, "entries": [{"id": "x", "tokens": toks[20:48], "want": [27]}, {"id": "y", "tokens": toks[:7], "want": [0, 6]}], "end": []},
        {"step": 3, "entries": [{"id": "x", "tokens": toks[48:49], "want": [0]}], "end": []},
        {"step": 4, "entries": [{"id": "x", "tokens": toks[49:50], "want": [0]}], "end": ["x", "y"]},
    ]
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
        out = replay(name, dtype, steps, tmp_path / dtype, max_tokens=128)
        want = plain_logits(name, 50, 3, dtype == "bfloat16").numpy()
        scale = np.abs(want).max()
        assert sorted(out) == [1, 2, 3, 4]
        assert np.abs(out[2][0] - want[47]).max() <= tol * scale
        assert np.abs(out[3][0] - want[48]).max() <= tol * scale and np.abs(out[4][0] - want[49]).max() <= tol * scale
        assert np.abs(out[1][0] - want[6]).max() <= tol * scale                 # the prompt's first 7 tokens are x's first 7
        assert np.abs(out[2][1] - want[0]).max() <= tol * scale and np.abs(out[2][2] - want[6]).max() <= tol * scale
        assert np.array_equal(out[1][0], out[2][2])                              # y's second life equals its first


def test_replay_refuses_bad_weights(tmp_path):
    import shutil
    from llmx_amd.weights import write_safetensors
    from llmx_amd.weights.folder import random_tensors
    from llmx_amd import MiniMaxM3Config
    from helpers import INIT_A, TINY_A
    folder = tmp_path / "broken"
    shutil.copytree(model_folder("A"), folder)
    tensors = random_tensors(MiniMaxM3Config(**TINY_A), INIT_A)
    del tensors["lm_head.weight"]
    tensors["model.extra.weight"] = torch.zeros(2)
    write_safetensors(folder / "model.safetensors", tensors)
    run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(tmp_path / "o"),
                          "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=120)
    assert run.returncode != 0
    assert "missing (1): lm_head.weight" in run.stderr and "unexpected (1): model.extra.weight" in run.stderr
