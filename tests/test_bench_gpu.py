"""bench.py's record: one JSON line with the fields its contract names, flat where the record keeps no deeper levels."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_one_line_and_exit_status_2():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 2 and len(run.stdout.strip().split("\n")) == 1 and "one GPU" in run.stdout


def test_the_record_of_one_real_layer():
    """The default run's record at one layer of the real sizes (a few seconds): every field of the contract, the
    configuration flat with at most 20 keys and both numbers of layers, every point with its time, bytes, experts and
    fraction, the prefill with its flops and HBM fractions, fractions that follow from the other fields."""
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "1", "--steps", "3", "--warmup", "1", "--no-calibration"],
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.strip().split("\n") if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key, want in (("unit", "tok/s"), ("n_gpus", 1), ("steps", 3), ("warmup", 1), ("higher_is_better", True), ("scaling", "weak"),
                      ("dtype", "bf16"), ("vs_baseline", None)):
        assert rec[key] == want, key
    assert "decode tok/s" in rec["metric"] and "synthetic" in rec["data"]
    assert abs(rec["value"] - 8 * 1e3 / rec["ms_per_step"]) < 0.01 * rec["value"]
    cfg = rec["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert (cfg["layers"], cfg["layers_of_config"], cfg["global_batch"], cfg["seq_len"], cfg["hidden"], cfg["experts"], cfg["vocab"]) == \
        (1, 24, 8, 4096, 3072, 256, 200064)
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(roof["achieved"] - roof["bytes_gb"] / rec["ms_per_step"] * 1e3) < 0.01 * roof["achieved"]
    pts = rec["points"]
    assert len(pts) <= 20 and all(not isinstance(v, (dict, list)) for v in pts.values())
    for b in (1, 8, 64):
        for suffix in ("", "_ms", "_gb", "_experts", "_frac"):
            assert pts[f"decode_b{b}{suffix}"] > 0
        assert abs(pts[f"decode_b{b}"] - b * 1e3 / pts[f"decode_b{b}_ms"]) < 0.01 * pts[f"decode_b{b}"]
        assert abs(pts[f"decode_b{b}_frac"] - pts[f"decode_b{b}_gb"] / pts[f"decode_b{b}_ms"] / 8.0) < 2e-3
    assert pts["decode_b1_experts"] == 8.0 and 8.0 < pts["decode_b8_experts"] <= 64.0 and pts["decode_b64_experts"] <= 256.0
    assert pts["decode_b8_logits_to_host"] > 0 and pts["generate_b8"] > 0 and 1.0 <= pts["generate_b8_rows_a_step"] <= 8.0
    pre = rec["prefill"]
    assert pre["tokens"] == 2048 and abs(pre["value"] - 2048 * 1e3 / pre["ms"]) < 0.01 * pre["value"]
    assert abs(pre["frac"] - pre["tflop"] * 1e12 / (pre["ms"] * 1e-3) / 2.5e15) < 2e-3
    assert 0 < pre["hbm_frac"] < 1 and pre["first_layer_experts"] > 200 and 0 < pre["first_layer_hbm_frac"] < 1
    # the bytes a step has to read, written out here for batch 8 at one layer: the attention's four projections, the
    # router, bias and norm weights in float32, the experts the step touched (three matrices each), the head and the
    # final norm, eight embedding rows, and keys and values of eight requests at the mean context of the timed steps
    experts = pts["decode_b8_experts"]
    want_bytes = ((6144 + 2 * 1024) * 3072 * 2 + 3072 * 6144 * 2            # q, k, v and o projections in bfloat16
                  + 256 * 3072 * 4 + 256 * 4                               # router matrix and correction bias in float32
                  + (2 * 3072 + 6144 + 1024) * 4                           # two layer norms, the q and k projection norms
                  + experts * 3 * 1536 * 3072 * 2                          # gate, up and down of each distinct expert
                  + 200064 * 3072 * 2 + 3072 * 4                           # head and final norm
                  + 8 * 3072 * 2                                           # embedding rows
                  + 8 * (4096 - 3 / 2) * 2 * 1024 * 2)                     # keys and values of 8 requests (8 heads of 128)
    assert abs(pts["decode_b8_gb"] - want_bytes / 1e9) <= 0.006, (pts["decode_b8_gb"], want_bytes / 1e9)
    assert roof["bytes_gb"] == pts["decode_b8_gb"]
    sw = rec["sweep"]
    assert all(not isinstance(v, (dict, list)) for v in sw.values())
    for name in ("decode_b8_ctx16384", "decode_b8_ctx32768", "decode_b16_ctx4096", "decode_b32_ctx4096", "decode_b128_ctx4096",
                 "decode_b64_ctx8192"):
        assert sw[name] > 0 and sw[name + "_ms"] > 0 and 0 < sw[name + "_frac"] < 1
    assert sw["mixed_512_beside_8_ms"] > 0
    assert sw["generate_b1"] > 0 and sw["generate_b1_ms"] > 0 and 0 < sw["generate_b1_frac"] < 1
    assert sw["prefill_8192"] > 0 and sw["prefill_8192_ms"] > 0 and 0 < sw["prefill_8192_frac"] < 1
    # 64 short prompts of different tokens pick most of the 256 experts, where one long prompt's rows pick few
    assert sw["prefill_spread_ms"] > 0 and sw["prefill_spread_experts"] > 150 and 0 < sw["prefill_spread_frac"] < 1
    assert "long" not in rec        # the long-context configuration belongs to the default run only
