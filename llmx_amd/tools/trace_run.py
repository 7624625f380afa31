"""Trace replay: feeds given token ids through a model step by step and writes logits.  It samples nothing.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps are read from standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one batch through the engine's own step function (the model, cache and kernels that
generation uses).  For a step in which something is wanted the logits at the wanted places are written to
OUT/<step>.f32 as little-endian float32 [wanted, vocab], in the order of the entries and of `want`.  After every step
`done <step>` is printed and flushed.  Requests named in `end` give back what they hold after the step.
With --routing the routed layers' expert picks and router logits of every step's rows are written beside the logits
(OUT/<step>.picks.i32 [routed layers, rows, k], OUT/<step>.router.f32 [routed layers, rows, experts]), as the reference's
route hook shows them (/root/reference/src/model/arch/blocks.hpp:118-138).
Modelled on the reference's captures (/root/reference/tools/model_logits.cpp:82-109) and its replay of recorded passes
(/root/reference/src/server/scheduler.hpp:860-868).
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each request's count rounded up to a multiple of 64")
    ap.add_argument("--page-tokens", type=int, default=16, help="tokens a cache page holds")
    ap.add_argument("--max-requests", type=int, default=8, help="most requests live at a time")
    ap.add_argument("--routing", action="store_true", help="also write every step's expert picks and router logits")
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    if args.page_tokens <= 0:
        ap.error("--page-tokens must be positive")

    out = Path(args.out)
    out.mkdir(parents=True, exist_ok=True)

    import numpy as np
    from llmx_amd.engine import Engine, StepEntry

    # --max-tokens counts each request rounded up to a multiple of 64 (to the engine's own page where that is larger).
    # A request of n tokens holds ceil(n / page) pages, which for pages that do not divide 64 can be one page more than
    # its rounded count holds; one page a request on top covers that for any page size.
    unit = max(64, args.page_tokens)
    kv_tokens = -(-args.max_tokens // unit) * unit
    if unit % args.page_tokens:
        kv_tokens += args.max_requests * args.page_tokens
    engine = Engine.load(args.model, dtype=args.dtype, kv_tokens=kv_tokens, page_tokens=args.page_tokens,
                         max_requests=args.max_requests)
    routed = []      # what the routed layers of the running step showed, in run order
    if args.routing:
        def observer(step, kind, **tensors):
            if kind == "routing":
                routed.append((tensors["ids"].cpu().numpy().copy(), tensors["logits"].cpu().numpy().copy()))
        engine.observer = observer
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step_no = record["step"]
        entries = []
        for e in record.get("entries", []):
            rid = e["id"]
            if not engine.has_request(rid):
                engine.add_request(rid)
            entries.append(StepEntry(rid, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if entries:
            routed.clear()
            logits = engine.step(entries)
            if routed:
                np.stack([ids for ids, _ in routed]).astype("<i4").tofile(out / f"{step_no}.picks.i32")
                np.stack([z for _, z in routed]).astype("<f4").tofile(out / f"{step_no}.router.f32")
            if logits.shape[0]:
                host = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                host.tofile(out / f"{step_no}.f32")
        for rid in record.get("end", []):
            if engine.has_request(rid):
                engine.end_request(rid)
        print(f"done {step_no}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
