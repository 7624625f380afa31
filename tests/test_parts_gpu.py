"""Each part alone against its plain formula, and the generality of the assembly: a toy mixer with state of its own,
defined here, registered, built and stepped without a change to the framework; a run order that names a layer twice
and lets a layer read another layer's cache; attention with a window whose pages are given back."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def make_step(dtype, entries, tables=(), page_tokens=4):
    """A StepState as the engine makes it: entries = [(slot, n, past)]."""
    from llmx_amd.engine.batch import EntryView, StepState, Workspace
    step = StepState(Workspace(DEV), dtype)
    views, row0 = [], 0
    for i, (slot, n, past) in enumerate(entries):
        views.append(EntryView(i, slot, row0, n, past))
        row0 += n
    step.rows = row0
    step.entries = views
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    step.positions = i32([v.past + r for v in views for r in range(v.n)])
    step.row_entry = i32([i for i, v in enumerate(views) for _ in range(v.n)])
    step.entry_slots = i32([v.slot for v in views])
    step.token_ids = i32([0] * row0)
    step._tables = [i32(t) for t in tables]
    return step


def ctx(dtype, max_positions=256, page_tokens=None):
    from llmx_amd.parts import BuildContext
    return BuildContext(dtype, DEV, max_positions, page_tokens)


def load_part(part, w):
    """Hands a part the tensors `w` (by the names it lists) as the loader does: on the device, a tensor that is a slice
    of a fused one (TensorSpec.into) copied into its place there."""
    out = {}
    for s in part.tensor_specs(set(w)):
        if s.into is None:
            out[s.name] = w[s.name].to(DEV)
        else:
            target, shape, index = s.into
            if target not in out:
                out[target] = torch.empty(shape, dtype=w[s.name].dtype, device=DEV)
            out[target][index].copy_(w[s.name])
    part.load(out)


def rnd(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return torch.randn(*shape, generator=g) * scale


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_embedding_head_parts(dtype):
    from llmx_amd.parts import PartSpec, build_part
    c = ctx(dtype)
    norm = build_part("norm", PartSpec("rmsnorm", {"width": 40, "eps": 1e-5}, "n."), c)
    assert [(s.name, s.shape, s.role) for s in norm.tensor_specs(set())] == [("n.weight", (40,), "norm")]
    w = 1 + 0.1 * rnd(40)
    norm.load({"n.weight": w.to(DEV)})
    x = rnd(5, 40, seed=1).to(DEV)
    step = make_step(dtype, [(0, 5, 0)])
    out = torch.empty(5, 40, dtype=dtype, device=DEV)
    out32 = torch.empty(5, 40, dtype=torch.float32, device=DEV)
    norm.forward(step, x, out, out32)
    want = pm.rms_norm(x.double().cpu(), w.double(), 1e-5)
    assert (out32.double().cpu() - want).abs().max() < 1e-5 and torch.equal(out, out32.to(dtype))

    emb = build_part("embedding", PartSpec("token_embedding", {"vocab": 30, "hidden": 40}, "e."), c)
    table = rnd(30, 40, seed=2).to(dtype).to(DEV)
    emb.load({"e.weight": table})
    step.token_ids = torch.tensor([3, 29, 0, 3, 7], dtype=torch.int32, device=DEV)
    xe = torch.empty(5, 40, dtype=torch.float32, device=DEV)
    emb.forward(step, xe)
    assert torch.equal(xe, table[step.token_ids.long()].float())

    head = build_part("head", PartSpec("linear", {"vocab": 30, "hidden": 40, "tied": True}, "h."), c)
    assert head.tensor_specs(set()) == []
    head.tie(emb.table())
    rows = rnd(2, 40, seed=3).to(dtype).to(DEV)
    logits = torch.empty(2, 30, dtype=torch.float32, device=DEV)
    head.forward(step, rows, logits)
    want = rows.double().cpu() @ table.double().cpu().T
    assert (logits.double().cpu() - want).abs().max() < 1e-4 * want.abs().max()


def test_position_part_equals_the_plain_tables():
    """The engine's rotary table and the plain implementation's share no code and agree bit for bit."""
    from llmx_amd.parts import PartSpec, build_part
    for R, theta, D in ((8, 1e4, 16), (24, 1e6, 24), (64, 5e6, 128)):
        pos = build_part("position", PartSpec("rotary_neox_partial", {"rotary_dim": R, "theta": theta, "head_dim": D}), ctx(torch.float32, 5000))
        table, rotary = pos.rotation()
        cos, sin = pm.rope_tables(list(range(5000)), R, theta)
        assert rotary == R and torch.equal(table.cpu(), torch.cat([cos, sin], dim=1))
    none = build_part("position", PartSpec("none"), ctx(torch.float32, 10))
    assert none.rotation()[1] == 0
    with pytest.raises(ValueError, match="rotary width"):
        build_part("position", PartSpec("rotary_neox_partial", {"rotary_dim": 20, "theta": 1e4, "head_dim": 16}), ctx(torch.float32))


@pytest.mark.parametrize("dtype,page", [(torch.float32, 4), (torch.bfloat16, 4), (torch.bfloat16, 16)])
@pytest.mark.parametrize("heads,kv_heads,D,R,qk_norm", [(4, 2, 16, 8, "projection"), (6, 1, 32, 32, "none")])
def test_attention_part(dtype, page, heads, kv_heads, D, R, qk_norm):
    """The mixer alone over two steps (a prompt portion, then the rest beside another request's first tokens)."""
    from llmx_amd.parts import LayerCache, PartSpec, build_part
    E, L1, L2 = 48, 37, 6
    params = {"hidden": E, "heads": heads, "kv_heads": kv_heads, "head_dim": D, "qk_norm": qk_norm, "eps": 1e-5, "window": None,
              "position": PartSpec("rotary_neox_partial", {"rotary_dim": R, "theta": 1e4, "head_dim": D})}
    att = build_part("mixer", PartSpec("attention", params, "a."), ctx(dtype))
    need = att.cache_need()
    assert need.window is None and [(t.name, t.shape, t.dtype, t.page_shape(page)) for t in need.tensors] == \
        [("k", (kv_heads, D), None, (kv_heads, page, D)), ("v", (kv_heads, D), None, (kv_heads, D, page))]
    w = {}
    for s in att.tensor_specs(set()):
        t = (1 + 0.1 * rnd(*s.shape, seed=len(w))) if s.role == "norm" else rnd(*s.shape, scale=0.3, seed=len(w))
        w[s.name] = t.to(torch.float32 if s.role == "norm" else dtype)
    load_part(att, w)
    n_pages = 16
    cache = LayerCache(group=0, tensors={"k": torch.zeros(n_pages, kv_heads, page, D, dtype=dtype, device=DEV),
                                         "v": torch.zeros(n_pages, kv_heads, D, page, dtype=dtype, device=DEV)}, writes=True)
    h1, h2 = rnd(L1, E, seed=5), rnd(L2, E, seed=6)
    pages1 = list(range(3, 3 + -(-L1 // page)))[::-1]           # out of order on purpose
    pages2 = [0, 1, 2][: -(-L2 // page)]
    width = 12
    row = lambda p: p + [-1] * (width - len(p))
    cut = 21
    got = []
    # step 1: the first 21 rows of request 1
    step = make_step(dtype, [(0, cut, 0)], [[row(pages1)]], page)
    out = torch.zeros(cut, E, dtype=torch.float32, device=DEV)
    att.forward(step, h1[:cut].to(dtype).to(DEV), out, False, cache)
    got.append(out.cpu())
    # step 2: the rest of request 1 beside all of request 2; accumulate into a residual
    step = make_step(dtype, [(0, L1 - cut, cut), (1, L2, 0)], [[row(pages1), row(pages2)]], page)
    base = rnd(L1 - cut + L2, E, seed=7)
    out = base.clone().to(DEV)
    att.forward(step, torch.cat([h1[cut:], h2]).to(dtype).to(DEV), out, True, cache)
    got.append((out.cpu() - base))
    cfg = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": D, "rms_norm_eps": 1e-5, "rotary_dim": R,
           "rope_parameters": {"rope_theta": 1e4}}
    rt = None if dtype == torch.float32 else torch.bfloat16
    wd = {k: v.double() for k, v in w.items()}
    if qk_norm == "none":
        wd["a.q_norm.weight"] = torch.ones(heads * D, dtype=torch.float64)
        wd["a.k_norm.weight"] = torch.ones(kv_heads * D, dtype=torch.float64)
        cfg["rms_norm_eps"] = 0.0

        def no_norm(x, weight, eps):
            return x
        real = pm.rms_norm
        pm.rms_norm = no_norm
    try:
        want1 = pm.attention_layer(pm._rounded(h1.double(), rt), list(range(L1)), wd, "a.", cfg, rt)
        want2 = pm.attention_layer(pm._rounded(h2.double(), rt), list(range(L2)), wd, "a.", cfg, rt)
    finally:
        if qk_norm == "none":
            pm.rms_norm = real
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    scale = want1.abs().max()
    assert (got[0].double() - want1[:cut]).abs().max() <= tol * scale
    assert (got[1][:L1 - cut].double() - want1[cut:]).abs().max() <= tol * scale
    assert (got[1][L1 - cut:].double() - want2).abs().max() <= tol * want2.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [3, 200])
def test_routed_experts_and_dense_glu_parts(dtype, T):
    from llmx_amd.parts import PartSpec, build_part
    E, X, k, Fe = 40, 12, 3, 24
    moe = build_part("feed_forward", PartSpec("routed_experts", {"hidden": E, "experts": X, "top_k": k, "intermediate": Fe, "score": "sigmoid",
                                                                 "correction_bias": True, "normalize": False, "scale": 1.5}, "m."), ctx(dtype))
    assert moe.wants_f32_input
    w = {}
    for s in moe.tensor_specs(set()):
        w[s.name] = rnd(*s.shape, scale=0.3 if s.role != "bias" else 0.1, seed=len(w)).to(torch.float32 if s.role in ("router", "bias") else dtype)
    moe.load({n: t.to(DEV) for n, t in w.items()})
    h = rnd(T, E, seed=9)
    step = make_step(dtype, [(0, T, 0)])
    seen = {}
    step.observer = lambda st, kind, **t: seen.update({kind: {n: v.clone() for n, v in t.items()}})
    out = torch.zeros(T, E, dtype=torch.float32, device=DEV)
    moe.forward(step, h.to(dtype).to(DEV), out, False, h.to(DEV))
    cfg = dict(num_experts_per_tok=k, norm_topk_prob=False, routed_scaling_factor=1.5)
    rt = None if dtype == torch.float32 else torch.bfloat16
    wd = {n: t.double() for n, t in w.items()}
    # the router reads the unrounded rows; the experts read the rounded ones
    z = h.double() @ wd["m.gate.weight"].T
    ids, weights = pm.route(z, wd["m.gate.e_score_correction_bias"], k, False, 1.5)
    assert torch.equal(seen["routing"]["ids"].long().cpu(), ids)
    hin = pm._rounded(h.double(), rt)
    want = torch.zeros(T, E, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            want[t] += weights[t, j] * pm.swiglu_expert(hin[t], wd["m.experts.gate_up_proj"][e], wd["m.experts.down_proj"][e], rt)
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    assert (out.double().cpu() - want).abs().max() <= tol * want.abs().max()

    glu = build_part("feed_forward", PartSpec("dense_glu", {"hidden": E, "intermediate": Fe}, "g."), ctx(dtype))
    gw = {s.name: rnd(*s.shape, scale=0.3, seed=3 + i).to(dtype) for i, s in enumerate(glu.tensor_specs(set()))}
    load_part(glu, gw)
    base = rnd(T, E, seed=4)
    out = base.clone().to(DEV)
    glu.forward(step, h.to(dtype).to(DEV), out, True)
    gate_up = torch.cat([gw["g.gate_proj.weight"], gw["g.up_proj.weight"]]).double()
    want = base.double() + pm.swiglu_expert(hin, gate_up, gw["g.down_proj.weight"].double(), rt)
    assert (out.double().cpu() - want).abs().max() <= tol * want.abs().max()


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_position_encoding_defined_here_serves_the_attention_part(dtype):
    """Another position encoding (positions squeezed by a factor before the rotation, over the whole head), registered
    from outside the framework: the attention part takes it by name."""
    from llmx_amd.parts import LayerCache, PartSpec, build_part
    from llmx_amd.parts.base import PositionEncoding, register, unregister

    def squeezed_tables(n, R, theta, factor):
        i = torch.arange(R // 2, dtype=torch.float64)
        freq = 1.0 / theta ** (2.0 * i / R)
        angle = (torch.arange(n, dtype=torch.float64) / factor)[:, None] * freq[None, :]
        return torch.cos(angle), torch.sin(angle)

    class SqueezedRotary(PositionEncoding):
        def __init__(self, params, prefix, c):
            super().__init__(params, prefix, c)
            self.R = int(params["head_dim"])
            cos, sin = squeezed_tables(c.max_positions, self.R, float(params["theta"]), float(params["factor"]))
            self.cos_sin = torch.cat([cos, sin], dim=1).float().to(c.device)

        def rotation(self):
            return self.cos_sin, self.R

    register("position", "toy_squeezed_rotary", SqueezedRotary, replace=True)
    try:
        E, heads, kv_heads, D, L, page = 32, 4, 2, 16, 29, 4
        params = {"hidden": E, "heads": heads, "kv_heads": kv_heads, "head_dim": D, "qk_norm": "none", "eps": 1e-5, "window": None,
                  "position": PartSpec("toy_squeezed_rotary", {"head_dim": D, "theta": 100.0, "factor": 4.0})}
        att = build_part("mixer", PartSpec("attention", params, "a."), ctx(dtype))
        w = {s.name: rnd(*s.shape, scale=0.3, seed=i).to(dtype) for i, s in enumerate(att.tensor_specs(set()))}
        load_part(att, w)
        cache = LayerCache(group=0, tensors={"k": torch.zeros(8, kv_heads, page, D, dtype=dtype, device=DEV),
                                             "v": torch.zeros(8, kv_heads, D, page, dtype=dtype, device=DEV)}, writes=True)
        h = rnd(L, E, seed=11).to(dtype)
        step = make_step(dtype, [(0, L, 0)], [[[7, 6, 5, 4, 3, 2, 1, 0]]], page)
        out = torch.zeros(L, E, dtype=torch.float32, device=DEV)
        att.forward(step, h.to(DEV), out, False, cache)
        rt = None if dtype == torch.float32 else torch.bfloat16
        hd = h.double()
        q = (hd @ w["a.q_proj.weight"].double().T).view(L, heads, D)
        k = (hd @ w["a.k_proj.weight"].double().T).view(L, kv_heads, D)
        v = (hd @ w["a.v_proj.weight"].double().T).view(L, kv_heads, D)
        cos, sin = squeezed_tables(L, D, 100.0, 4.0)
        q, k = pm.apply_partial_rope(q, cos, sin, D), pm.apply_partial_rope(k, cos, sin, D)
        q, k, v = (pm._rounded(t, rt) for t in (q, k, v))
        o = pm._rounded(pm.causal_attention(q, k, v, None).reshape(L, heads * D), rt)
        want = o @ w["a.o_proj.weight"].double().T
        assert (out.double().cpu() - want).abs().max() <= (3e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    finally:
        unregister("position", "toy_squeezed_rotary")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_routed_feed_forward_defined_here(dtype):
    """A feed-forward with routing of its own (the expert is chosen by the row's position, one expert a row, weight 1),
    made outside the framework from its grouped products: registered, built, loaded by tensor name and run."""
    from llmx_amd import ops
    from llmx_amd.parts import PartSpec, TensorSpec, build_part
    from llmx_amd.parts.base import FeedForward, register, unregister

    class ByPosition(FeedForward):
        def __init__(self, params, prefix, c):
            super().__init__(params, prefix, c)
            self.E, self.X, self.F = int(params["hidden"]), int(params["experts"]), int(params["intermediate"])

        def tensor_specs(self, available):
            return [TensorSpec(self.name("up"), (self.X, 2 * self.F, self.E)), TensorSpec(self.name("down"), (self.X, self.E, self.F))]

        def load(self, tensors):
            self.up, self.down = tensors[self.name("up")], tensors[self.name("down")]

        def forward(self, step, h, out, accumulate, h32=None):
            T, X = step.rows, self.X
            ids = (step.positions % X).to(torch.int32).view(T, 1).contiguous()
            weights = torch.ones(T, 1, dtype=torch.float32, device=h.device)
            i32 = lambda name, n: step.buf("toy." + name, (n,), torch.int32)
            counts, offsets, pairs, active, n_active = i32("counts", X), i32("offsets", X + 1), i32("pairs", T), i32("active", X), i32("n", 1)
            ops.moe_align(ids, X, counts, offsets, pairs, active, n_active)
            act = step.buf("toy.act", (T, self.F), step.act_dtype)
            ops.grouped_gemm(h, self.up, act, offsets, pairs, 1, ops.EPI_SWIGLU, active, n_active, token_rows=T)
            y = step.buf("toy.y", (T, self.E), torch.float32)
            ops.grouped_gemm(act, self.down, y, offsets, pairs, 1, ops.EPI_STORE, active, n_active, token_rows=T)
            ops.moe_combine(out, y, ids, weights, accumulate)

    register("feed_forward", "toy_by_position", ByPosition, replace=True)
    try:
        E, X, Fe = 40, 5, 24
        for T, past in ((3, 0), (70, 9)):
            ff = build_part("feed_forward", PartSpec("toy_by_position", {"hidden": E, "experts": X, "intermediate": Fe}, "t."), ctx(dtype))
            assert not ff.graph_safe
            w = {s.name: rnd(*s.shape, scale=0.3, seed=i).to(dtype) for i, s in enumerate(ff.tensor_specs(set()))}
            ff.load({n: t.to(DEV) for n, t in w.items()})
            h = rnd(T, E, seed=5).to(dtype)
            step = make_step(dtype, [(0, T, past)])
            base = rnd(T, E, seed=6)
            out = base.clone().to(DEV)
            ff.forward(step, h.to(DEV), out, True)
            rt = None if dtype == torch.float32 else torch.bfloat16
            want = base.double().clone()
            for t in range(T):
                e = (past + t) % X
                want[t] += pm.swiglu_expert(h[t].double(), w["t.up"][e].double(), w["t.down"][e].double(), rt)
            assert (out.double().cpu() - want).abs().max() <= (3e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    finally:
        unregister("feed_forward", "toy_by_position")


# ---------------------------------------------------------------------------
# A toy architecture made here: layers alternate attention and a mixer that keeps a running state per request.
ToyState = None


def define_toy_parts():
    from llmx_amd.parts import Mixer, StateNeed, TensorSpec, register

    class RunningMean(Mixer):
        """out_t = s_t with s_t = decay * s_{t-1} + (1 - decay) * (h_t @ W^T); the state s lives in the request's slot."""
        wants_f32_input = True

        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.hidden = params["hidden"]
            self.decay = params["decay"]
            self.weight = None

        def cache_need(self):
            return StateNeed((self.hidden,), "float32")

        def tensor_specs(self, available):
            return [TensorSpec(self.name("mix.weight"), (self.hidden, self.hidden), "router")]   # kept in float32

        def load(self, tensors):
            self.weight = tensors[self.name("mix.weight")]

        fail_after_writing = False     # set by a test: the step dies once this layer has written its state

        def forward(self, step, h, out, accumulate, cache, h32=None):
            y = h32 @ self.weight.T
            result = torch.empty_like(y)
            for e in step.entries:                      # each request's rows in order, from and to its own slot
                s = cache.state[e.slot]
                for r in range(e.row0, e.row0 + e.n):
                    s = self.decay * s + (1.0 - self.decay) * y[r]
                    result[r] = s
                cache.state[e.slot] = s
            if self.fail_after_writing:
                raise RuntimeError("the toy mixer was told to fail")
            if accumulate:
                out += result
            else:
                out.copy_(result)

    register("mixer", "toy_running_mean", RunningMean, replace=True)
    return RunningMean


@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int = 50
    hidden_size: int = 32
    layers: int = 4
    decay: float = 0.75
    architecture = "ToyHybridForCausalLM"

    @classmethod
    def from_json(cls, values):
        return cls(**{k: v for k, v in values.items() if k != "architectures"})

    def to_json(self):
        return {"architectures": [self.architecture], "vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "layers": self.layers,
                "decay": self.decay}


def toy_assemble(c: ToyConfig):
    from llmx_amd.parts import BlockSpec, ModelSpec, PartSpec, RunEntry
    E = c.hidden_size
    blocks = []
    for i in range(c.layers):
        p = f"layers.{i}."
        norm = {"width": E, "eps": 1e-5}
        if i % 2 == 0:
            mixer = PartSpec("attention", {"hidden": E, "heads": 4, "kv_heads": 2, "head_dim": 8, "qk_norm": "none",
                                           "position": PartSpec("rotary_neox_partial", {"rotary_dim": 4, "theta": 100.0, "head_dim": 8})}, p + "attn.")
        else:
            mixer = PartSpec("toy_running_mean", {"hidden": E, "decay": c.decay}, p + "toy.")
        ffn = PartSpec("dense_glu", {"hidden": E, "intermediate": 24}, p + "mlp.")
        blocks.append(BlockSpec(PartSpec("rmsnorm", norm, p + "n1."), mixer, PartSpec("rmsnorm", norm, p + "n2."), ffn))
    return ModelSpec(architecture=c.architecture, vocab_size=c.vocab_size, hidden_size=E, max_positions=128,
                     embedding=PartSpec("token_embedding", {"vocab": c.vocab_size, "hidden": E}, "embed."), blocks=blocks,
                     run_order=[RunEntry(i, i) for i in range(c.layers)], final_norm=PartSpec("rmsnorm", {"width": E, "eps": 1e-5}, "norm."),
                     head=PartSpec("linear", {"vocab": c.vocab_size, "hidden": E, "tied": True}, "head."))


def toy_plain(weights, c: ToyConfig, tokens):
    """The toy model's formulas, whole sequence, float64."""
    x = weights["embed.weight"].double()[tokens]
    T = len(tokens)
    for i in range(c.layers):
        p = f"layers.{i}."
        h = pm.rms_norm(x, weights[p + "n1.weight"].double(), 1e-5)
        if i % 2 == 0:
            q = (h @ weights[p + "attn.q_proj.weight"].double().T).view(T, 4, 8)
            k = (h @ weights[p + "attn.k_proj.weight"].double().T).view(T, 2, 8)
            v = (h @ weights[p + "attn.v_proj.weight"].double().T).view(T, 2, 8)
            cos, sin = pm.rope_tables(list(range(T)), 4, 100.0)
            q, k = pm.apply_partial_rope(q, cos, sin, 4), pm.apply_partial_rope(k, cos, sin, 4)
            x = x + pm.causal_attention(q, k, v).reshape(T, 32) @ weights[p + "attn.o_proj.weight"].double().T
        else:
            y = h @ weights[p + "toy.mix.weight"].double().T
            s = torch.zeros(c.hidden_size, dtype=torch.float64)
            out = torch.zeros_like(y)
            for t in range(T):
                s = c.decay * s + (1 - c.decay) * y[t]
                out[t] = s
            x = x + out
        h = pm.rms_norm(x, weights[p + "n2.weight"].double(), 1e-5)
        gate_up = torch.cat([weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"]]).double()
        x = x + pm.swiglu_expert(h, gate_up, weights[p + "mlp.down_proj.weight"].double())
    return pm.rms_norm(x, weights["norm.weight"].double(), 1e-5) @ weights["embed.weight"].double().T


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    """Nothing in llmx_amd changes: the part and the architecture are registered from here."""
    import json
    from llmx_amd import Engine, RandomInit
    from llmx_amd.engine import StepEntry
    from llmx_amd.models import register_architecture, unregister_architecture
    from llmx_amd.parts import StateNeed, unregister
    from llmx_amd.weights import write_safetensors
    from llmx_amd.weights.random_init import host_values
    define_toy_parts()
    register_architecture("ToyHybridForCausalLM", ToyConfig, toy_assemble, replace=True)
    try:
        c = ToyConfig()
        # a model folder written with the framework's own random-weights mode
        from llmx_amd.weights.folder import write_random_model
        folder = write_random_model(tmp_path / "toy", c, RandomInit(seed=4, std=0.2, norm_std=0.05, storage="float32"))
        assert json.loads((folder / "config.json").read_text())["architectures"] == ["ToyHybridForCausalLM"]
        engine = Engine.load(folder, dtype="float32", kv_tokens=64, page_tokens=4, max_requests=3)
        needs = engine.model.cache_needs()
        assert [type(n).__name__ for n in needs] == ["PagedNeed", "StateNeed", "PagedNeed", "StateNeed"]
        assert not engine.graphs, "a part that does not say graph_safe must keep the engine from recording graphs"
        weights, _ = {}, None
        from safetensors import safe_open
        with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
            weights = {n: f.get_tensor(n) for n in f.keys()}
        seqs = {"a": [3, 14, 15, 9, 2, 6, 5, 35, 8, 9, 7, 9, 3, 2, 38, 4, 6], "b": [2, 7, 18, 28, 18, 2, 8, 4, 5, 9, 0, 45]}
        want = {r: toy_plain(weights, c, t) for r, t in seqs.items()}
        # whole
        for r, t in seqs.items():
            engine.add_request(r)
            got = engine.step([StepEntry(r, t, list(range(len(t))))]).cpu().double()
            engine.end_request(r)
            assert (got - want[r]).abs().max() < 2e-5 * want[r].abs().max()
        # mixed: portions of one beside single tokens of the other; a slot reused by a new request starts from a zero state
        engine.add_request("a")
        engine.add_request("b")
        at = {"a": 0, "b": 0}
        rows = {"a": [], "b": []}
        plan = [(5, 1), (2, 1), (1, 3), (4, 1), (3, 2), (2, 4)]
        for na, nb in plan:
            entries = []
            for r, n in (("a", na), ("b", nb)):
                n = min(n, len(seqs[r]) - at[r])
                if n:
                    entries.append(StepEntry(r, seqs[r][at[r]:at[r] + n], list(range(n))))
            out = engine.step(entries).cpu().double()
            i = 0
            for e in entries:
                rows[e.request].append(out[i:i + len(e.tokens)])
                i += len(e.tokens)
                at[e.request] += len(e.tokens)
        for r in seqs:
            assert at[r] == len(seqs[r])
            assert (torch.cat(rows[r]) - want[r]).abs().max() < 2e-5 * want[r].abs().max()
        engine.end_request("a")
        engine.end_request("b")
        engine.add_request("c")       # takes a slot that held state
        got = engine.step([StepEntry("c", seqs["b"], list(range(len(seqs["b"]))))]).cpu().double()
        assert (got - want["b"]).abs().max() < 2e-5 * want["b"].abs().max()
    finally:
        unregister_architecture("ToyHybridForCausalLM")
        unregister("mixer", "toy_running_mean")


def test_a_step_that_fails_leaves_the_state_as_it_found_it(tmp_path):
    """A step in which the stateful toy mixer has already written its state raises; the next step gives the bits of an
    engine that never failed: pages were returned and every request's state is what the last good step left."""
    from llmx_amd import Engine, RandomInit
    from llmx_amd.engine import StepEntry, StepError
    from llmx_amd.models import register_architecture, unregister_architecture
    from llmx_amd.parts import unregister
    from llmx_amd.weights.folder import write_random_model
    define_toy_parts()
    register_architecture("ToyHybridForCausalLM", ToyConfig, toy_assemble, replace=True)
    try:
        folder = write_random_model(tmp_path / "toy", ToyConfig(), RandomInit(seed=4, std=0.2, norm_std=0.05, storage="float32"))
        failing, steady = (Engine.load(folder, dtype="float32", kv_tokens=64, page_tokens=4, max_requests=2) for _ in range(2))
        a, b = [3, 14, 15, 9, 2, 6, 5, 35, 8, 9, 7, 9], [2, 7, 18, 28, 18, 2, 8]
        every = lambda t: list(range(len(t)))
        for eng in (failing, steady):
            eng.add_request("a")
            eng.add_request("b")
            eng.step([StepEntry("a", a[:5], []), StepEntry("b", b[:3], [])])
        pages = failing.cache.pages_in_use()
        slots = (failing.cache.slot("a"), failing.cache.slot("b"))
        last_toy = failing.model.blocks[3].mixer
        last_toy.fail_after_writing = True
        with pytest.raises(RuntimeError, match="told to fail"):
            failing.step([StepEntry("a", a[5:9], every(a[5:9])), StepEntry("b", b[3:4], [0])])
        last_toy.fail_after_writing = False
        assert failing.cache.pages_in_use() == pages and failing.length("a") == 5 and failing.length("b") == 3
        assert (failing.cache.slot("a"), failing.cache.slot("b")) == slots and failing.cache.slots.in_use == 2
        for cut in ([StepEntry("a", a[5:9], every(a[5:9])), StepEntry("b", b[3:4], [0])], [StepEntry("a", a[9:], every(a[9:])), StepEntry("b", b[4:], every(b[4:]))]):
            assert torch.equal(failing.step(cut), steady.step(cut))
        # a state cannot be unwound: taking a stateful request back to a prefix is refused, to nothing is allowed
        with pytest.raises(StepError, match="keeps a state of fixed size"):
            failing.truncate("a", 4)
        failing.truncate("a", 0)
        steady.end_request("a")
        steady.add_request("a")
        assert torch.equal(failing.step([StepEntry("a", a, every(a))]), steady.step([StepEntry("a", a, every(a))]))
    finally:
        unregister_architecture("ToyHybridForCausalLM")
        unregister("mixer", "toy_running_mean")


def test_an_arrangement_defined_here_with_norms_after_its_parts(tmp_path):
    """Another arrangement of a layer, registered from outside: norms after the mixer and after the feed-forward as well
    as before them (x += post(mixer(pre(x))); x += post(ffn(pre(x)))), the two further norms being extra parts of the
    block, and a softmax scale of the architecture's own.  Built, loaded from a folder and stepped in portions; compared
    with the formulas written out."""
    from dataclasses import dataclass as dc
    from llmx_amd import Engine, RandomInit
    from llmx_amd.engine import StepEntry
    from llmx_amd.models import register_architecture, unregister_architecture
    from llmx_amd.parts import BlockSpec, ModelSpec, PartSpec, RunEntry, build_part, register, unregister
    from llmx_amd.weights.folder import write_random_model
    from safetensors import safe_open

    class SandwichBlock:
        graph_safe = False      # it adds with a library call

        def __init__(self, spec, c):
            self.mixer_norm, self.mixer = build_part("norm", spec.mixer_norm, c), build_part("mixer", spec.mixer, c)
            self.ffn_norm, self.ffn = build_part("norm", spec.ffn_norm, c), build_part("feed_forward", spec.ffn, c)
            self.after = {name: build_part(family, part, c) for name, (family, part) in spec.extra.items()}

        def parts(self):
            return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, *self.after.values()]

        def forward(self, step, x, cache):
            T, E = x.shape
            h = step.buf("sandwich.h", (T, E), step.act_dtype)
            y = step.buf("sandwich.y", (T, E), torch.float32)
            y32 = step.buf("sandwich.y32", (T, E), torch.float32)
            for norm, part, post, is_mixer in ((self.mixer_norm, self.mixer, self.after["post_mixer_norm"], True),
                                               (self.ffn_norm, self.ffn, self.after["post_ffn_norm"], False)):
                norm.forward(step, x, h)
                if is_mixer:
                    part.forward(step, h, y, False, cache)
                else:
                    part.forward(step, h, y, False)
                post.forward(step, y, None, y32)
                x += y32

    @dc(frozen=True)
    class SandwichConfig:
        vocab_size: int = 40
        hidden_size: int = 32
        layers: int = 2
        architecture = "ToySandwichForCausalLM"

        @classmethod
        def from_json(cls, values):
            return cls(**{k: v for k, v in values.items() if k != "architectures"})

        def to_json(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "layers": self.layers}

    SCALE = 0.2

    def assemble(c):
        E = c.hidden_size
        norm = lambda prefix: PartSpec("rmsnorm", {"width": E, "eps": 1e-5}, prefix)
        blocks = []
        for i in range(c.layers):
            p = f"layers.{i}."
            mixer = PartSpec("attention", {"hidden": E, "heads": 4, "kv_heads": 2, "head_dim": 8, "qk_norm": "none", "scale": SCALE,
                                           "position": PartSpec("rotary_neox_partial", {"rotary_dim": 8, "theta": 100.0, "head_dim": 8,
                                                                                        "pairing": "interleaved"})}, p + "attn.")
            blocks.append(BlockSpec(norm(p + "n1."), mixer, norm(p + "n2."), PartSpec("dense_glu", {"hidden": E, "intermediate": 24}, p + "mlp."),
                                    arrangement="toy_sandwich",
                                    extra={"post_mixer_norm": ("norm", norm(p + "n1_post.")), "post_ffn_norm": ("norm", norm(p + "n2_post."))}))
        return ModelSpec(architecture=c.architecture, vocab_size=c.vocab_size, hidden_size=E, max_positions=64,
                         embedding=PartSpec("token_embedding", {"vocab": c.vocab_size, "hidden": E}, "embed."), blocks=blocks,
                         run_order=[RunEntry(i, i) for i in range(c.layers)], final_norm=norm("norm."),
                         head=PartSpec("linear", {"vocab": c.vocab_size, "hidden": E, "tied": True}, "head."))

    def interleaved_rope(x, positions, theta):
        """pairs (2j, 2j + 1) of each head rotated by position * theta^(-2j / D)"""
        D = x.shape[-1]
        j = torch.arange(D // 2, dtype=torch.float64)
        angle = torch.tensor(positions, dtype=torch.float64)[:, None] * (1.0 / theta ** (2.0 * j / D))[None, :]
        c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
        a, b = x[..., 0::2], x[..., 1::2]
        out = torch.empty_like(x)
        out[..., 0::2] = a * c - b * s
        out[..., 1::2] = b * c + a * s
        return out

    def plain(w, c, tokens):
        T = len(tokens)
        x = w["embed.weight"].double()[tokens]
        for i in range(c.layers):
            p = f"layers.{i}."
            h = pm.rms_norm(x, w[p + "n1.weight"].double(), 1e-5)
            q = interleaved_rope((h @ w[p + "attn.q_proj.weight"].double().T).view(T, 4, 8), list(range(T)), 100.0)
            k = interleaved_rope((h @ w[p + "attn.k_proj.weight"].double().T).view(T, 2, 8), list(range(T)), 100.0)
            v = (h @ w[p + "attn.v_proj.weight"].double().T).view(T, 2, 8)
            q = q * (SCALE * math.sqrt(8.0))         # causal_attention divides by sqrt(D): scores become q.k * SCALE
            y = pm.causal_attention(q, k, v).reshape(T, 32) @ w[p + "attn.o_proj.weight"].double().T
            x = x + pm.rms_norm(y, w[p + "n1_post.weight"].double(), 1e-5)
            h = pm.rms_norm(x, w[p + "n2.weight"].double(), 1e-5)
            gate_up = torch.cat([w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"]]).double()
            y = pm.swiglu_expert(h, gate_up, w[p + "mlp.down_proj.weight"].double())
            x = x + pm.rms_norm(y, w[p + "n2_post.weight"].double(), 1e-5)
        return pm.rms_norm(x, w["norm.weight"].double(), 1e-5) @ w["embed.weight"].double().T

    register("block", "toy_sandwich", SandwichBlock, replace=True)
    register_architecture("ToySandwichForCausalLM", SandwichConfig, assemble, replace=True)
    try:
        c = SandwichConfig()
        folder = write_random_model(tmp_path / "sandwich", c, RandomInit(seed=9, std=0.3, norm_std=0.1, storage="float32"))
        with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
            weights = {n: f.get_tensor(n) for n in f.keys()}
        assert "layers.1.n2_post.weight" in weights           # the extra parts' tensors are the model's
        tokens = [3, 14, 15, 9, 2, 6, 5, 35, 8, 9, 7, 9, 3, 2, 38, 4, 6, 2, 6]
        want = plain(weights, c, tokens)
        engine = Engine.load(folder, dtype="float32", kv_tokens=64, page_tokens=4, max_requests=2)
        engine.add_request("w")
        whole = engine.step([StepEntry("w", tokens, list(range(len(tokens))))]).clone()
        assert (whole.cpu().double() - want).abs().max() < 3e-5 * want.abs().max()
        engine.add_request("p")
        rows = [engine.step([StepEntry("p", tokens[a:b], list(range(b - a)))]).clone() for a, b in ((0, 7), (7, 9), (9, 18), (18, 19))]
        assert torch.equal(torch.cat(rows), whole)
    finally:
        unregister_architecture("ToySandwichForCausalLM")
        unregister("block", "toy_sandwich")


def test_run_order_names_a_layer_twice_and_shares_a_cache():
    """The run order is data: layer 1's weights run twice (with a cache each), and the last entry reads layer 0's cache."""
    from helpers import TINY_A, INIT_A, plain
    from llmx_amd import Engine, MiniMaxM3Config
    from llmx_amd.engine import StepEntry
    from llmx_amd.models import assemble
    from llmx_amd.parts import RunEntry
    from llmx_amd.weights import ModelFiles, load as load_weights
    from helpers import model_folder
    cfg = MiniMaxM3Config(**TINY_A)
    spec = assemble(cfg)
    spec.run_order = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(1, 2), RunEntry(0, 0, writes=False)]
    files = ModelFiles(model_folder("A"))
    engine = Engine(cfg, spec, "float32", kv_tokens=128, page_tokens=4, max_requests=2,
                    weights=lambda e: load_weights(e.model.tensor_specs(set(files.names())), files, e.device, True))
    assert len(engine._layer_caches) == 4 and engine._paged[0]["k"].shape[0] == 3
    tokens = [5, 17, 3, 200, 41, 7, 99, 1, 2, 3, 4]
    engine.add_request("w")
    whole = engine.step([StepEntry("w", tokens, list(range(len(tokens))))]).clone()
    engine.end_request("w")
    engine.add_request("p")
    parts = [engine.step([StepEntry("p", tokens[a:b], list(range(b - a)))]).clone() for a, b in ((0, 4), (4, 6), (6, 7), (7, 11))]
    assert torch.equal(torch.cat(parts), whole)
    # the plain implementation of the same order: layers 0, 1, 1, then layer 0's attention over the keys and values that
    # layer 0's first run wrote (its own k, v projections of the new input are not used)
    config, w = plain("A")
    x = w["model.embed_tokens.weight"].double()[tokens]
    T = len(tokens)
    kv0 = {}

    def layer(x, i, shared=None):
        p = f"model.layers.{i}."
        h = pm.rms_norm(x, w[p + "input_layernorm.weight"].double(), config["rms_norm_eps"])
        if shared is None:
            x = x + pm.attention_layer(h, list(range(T)), w, p + "self_attn.", config)
        else:
            q = pm.rms_norm(h @ w[p + "self_attn.q_proj.weight"].double().T, w[p + "self_attn.q_norm.weight"].double(), config["rms_norm_eps"])
            cos, sin = pm.rope_tables(list(range(T)), 8, 1e4)
            q = pm.apply_partial_rope(q.view(T, 4, 16), cos, sin, 8)
            x = x + pm.causal_attention(q, shared[0], shared[1]).reshape(T, 64) @ w[p + "self_attn.o_proj.weight"].double().T
        h = pm.rms_norm(x, w[p + "post_attention_layernorm.weight"].double(), config["rms_norm_eps"])
        return x + pm.moe_layer(h, w, p + "mlp.", config)[0]

    h0 = pm.rms_norm(x, w["model.layers.0.input_layernorm.weight"].double(), config["rms_norm_eps"])
    k0 = pm.rms_norm(h0 @ w["model.layers.0.self_attn.k_proj.weight"].double().T, w["model.layers.0.self_attn.k_norm.weight"].double(), config["rms_norm_eps"])
    cos, sin = pm.rope_tables(list(range(T)), 8, 1e4)
    k0 = pm.apply_partial_rope(k0.view(T, 2, 16), cos, sin, 8)
    v0 = (h0 @ w["model.layers.0.self_attn.v_proj.weight"].double().T).view(T, 2, 16)
    x = layer(x, 0)
    x = layer(x, 1)
    x = layer(x, 1)
    x = layer(x, 0, shared=(k0, v0))
    want = pm.rms_norm(x, w["model.norm.weight"].double(), config["rms_norm_eps"]) @ w["lm_head.weight"].double().T
    assert (whole.cpu().double() - want).abs().max() < 2e-5 * want.abs().max()


# ---------------------------------------------------------------------------
# A mixer whose cache is not keys and values: one float32 latent a token, in pages of its own group, and a parameter of
# a kind no role knows (a gain drawn uniformly from [0.5, 1.5), kept in float32 in both paths).
def define_latent_mixer():
    from llmx_amd.parts import CacheTensor, Mixer, PagedNeed, TensorSpec, register

    class LatentMixer(Mixer):
        """c_t = h_t Wc^T (a latent of `latent` values, cached); out_t = gain * ((sum_s<=t softmax_s(c_t . c_s / sqrt(latent)) c_s) Wo^T)."""
        wants_f32_input = True

        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.hidden, self.latent = params["hidden"], params["latent"]
            self.page = ctx.page_tokens
            self.wc = self.wo = self.gain = None

        def cache_need(self):
            return PagedNeed((CacheTensor("latent", (self.latent,), "float32", 0),))

        def tensor_specs(self, available):
            return [TensorSpec(self.name("down.weight"), (self.latent, self.hidden), "router"),
                    TensorSpec(self.name("up.weight"), (self.hidden, self.latent), "router"),
                    TensorSpec(self.name("gain"), (self.hidden,), "matrix", dtype="float32", init=("uniform", 0.5, 1.5))]

        def load(self, tensors):
            self.wc, self.wo, self.gain = (tensors[self.name(n)] for n in ("down.weight", "up.weight", "gain"))

        def forward(self, step, h, out, accumulate, cache, h32=None):
            # once a step, for every layer of this kind: each row's page and place in it, from the group's block tables
            def places():
                tables = step.tables(cache.group).cpu()
                page, slot = [], []
                for i, e in enumerate(step.entries):
                    for pos in range(e.past, e.past + e.n):
                        page.append(int(tables[i, pos // self.page]))
                        slot.append(pos % self.page)
                return torch.tensor(page, device=step.device), torch.tensor(slot, device=step.device), tables
            page, slot, tables = step.shared(("latent.places", cache.group), places)
            store = cache.tensors["latent"]                    # [pages, page_tokens, latent] float32
            assert store.dtype == torch.float32 and tuple(store.shape[1:]) == (self.page, self.latent)
            c = h32 @ self.wc.T
            if cache.writes:
                store[page, slot] = c
            result = torch.empty((step.rows, self.hidden), dtype=torch.float32, device=step.device)
            for i, e in enumerate(step.entries):
                n_ctx = e.past + e.n
                pages = tables[i, :-(-n_ctx // self.page)].to(step.device)
                ctx_latents = store[pages].reshape(-1, self.latent)[:n_ctx]
                scores = (c[e.row0:e.row0 + e.n] @ ctx_latents.T) / self.latent ** 0.5
                causal = torch.arange(n_ctx, device=step.device)[None, :] <= torch.arange(e.past, n_ctx, device=step.device)[:, None]
                weights = torch.softmax(scores.masked_fill(~causal, float("-inf")), dim=-1)
                result[e.row0:e.row0 + e.n] = ((weights @ ctx_latents) @ self.wo.T) * self.gain
            if accumulate:
                out += result
            else:
                out.copy_(result)

    register("mixer", "toy_latent", LatentMixer, replace=True)


@dataclass(frozen=True)
class LatentConfig:
    vocab_size: int = 40
    hidden_size: int = 32
    latent: int = 6
    layers: int = 4
    architecture = "ToyLatentForCausalLM"

    @classmethod
    def from_json(cls, values):
        return cls(**{k: v for k, v in values.items() if k != "architectures"})

    def to_json(self):
        return {"architectures": [self.architecture], "vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "latent": self.latent,
                "layers": self.layers}


def latent_assemble(c: LatentConfig):
    from llmx_amd.parts import BlockSpec, ModelSpec, PartSpec, RunEntry
    E = c.hidden_size
    blocks = []
    for i in range(c.layers):
        p = f"layers.{i}."
        norm = {"width": E, "eps": 1e-5}
        if i % 2 == 0:
            mixer = PartSpec("toy_latent", {"hidden": E, "latent": c.latent}, p + "latent.")
        else:
            mixer = PartSpec("attention", {"hidden": E, "heads": 4, "kv_heads": 2, "head_dim": 8, "qk_norm": "none"}, p + "attn.")
        blocks.append(BlockSpec(PartSpec("rmsnorm", norm, p + "n1."), mixer, PartSpec("rmsnorm", norm, p + "n2."),
                                PartSpec("dense_glu", {"hidden": E, "intermediate": 24}, p + "mlp.")))
    return ModelSpec(architecture=c.architecture, vocab_size=c.vocab_size, hidden_size=E, max_positions=128,
                     embedding=PartSpec("token_embedding", {"vocab": c.vocab_size, "hidden": E}, "embed."), blocks=blocks,
                     run_order=[RunEntry(i, i) for i in range(c.layers)], final_norm=PartSpec("rmsnorm", {"width": E, "eps": 1e-5}, "norm."),
                     head=PartSpec("linear", {"vocab": c.vocab_size, "hidden": E, "tied": True}, "head."))


def latent_plain(weights, c: LatentConfig, tokens):
    x = weights["embed.weight"].double()[tokens]
    T = len(tokens)
    for i in range(c.layers):
        p = f"layers.{i}."
        h = pm.rms_norm(x, weights[p + "n1.weight"].double(), 1e-5)
        if i % 2 == 0:
            lat = h @ weights[p + "latent.down.weight"].double().T
            scores = (lat @ lat.T) / c.latent ** 0.5
            scores = scores.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
            x = x + ((torch.softmax(scores, dim=-1) @ lat) @ weights[p + "latent.up.weight"].double().T) * weights[p + "latent.gain"].double()
        else:
            q = (h @ weights[p + "attn.q_proj.weight"].double().T).view(T, 4, 8)
            k = (h @ weights[p + "attn.k_proj.weight"].double().T).view(T, 2, 8)
            v = (h @ weights[p + "attn.v_proj.weight"].double().T).view(T, 2, 8)
            x = x + pm.causal_attention(q, k, v).reshape(T, 32) @ weights[p + "attn.o_proj.weight"].double().T
        h = pm.rms_norm(x, weights[p + "n2.weight"].double(), 1e-5)
        gate_up = torch.cat([weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"]]).double()
        x = x + pm.swiglu_expert(h, gate_up, weights[p + "mlp.down_proj.weight"].double())
    return pm.rms_norm(x, weights["norm.weight"].double(), 1e-5) @ weights["embed.weight"].double().T


def test_a_mixer_that_caches_one_latent_a_token_and_brings_a_parameter_of_its_own_kind(tmp_path):
    """The engine allocates what a mixer's need lists (here one float32 latent a token, where attention lists keys and
    values of the activation type), the loader and the random-weights mode follow what a tensor's spec states (a gain
    kept in float32, drawn uniformly from [0.5, 1.5)), and `step.shared` gives a part what it wants once a step: no file
    under llmx_amd changes for any of it."""
    from safetensors import safe_open
    from llmx_amd import Engine, RandomInit
    from llmx_amd.engine import StepEntry
    from llmx_amd.models import register_architecture, unregister_architecture
    from llmx_amd.parts import unregister
    from llmx_amd.weights.folder import write_random_model
    define_latent_mixer()
    register_architecture("ToyLatentForCausalLM", LatentConfig, latent_assemble, replace=True)
    try:
        c = LatentConfig()
        folder = write_random_model(tmp_path / "latent", c, RandomInit(seed=9, std=0.2, norm_std=0.05, storage="bfloat16"))
        with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
            weights = {n: f.get_tensor(n) for n in f.keys()}
        gain = weights["layers.0.latent.gain"]
        assert gain.dtype == torch.float32 and float(gain.min()) >= 0.5 and float(gain.max()) < 1.5 and float(gain.std()) > 0.2
        assert weights["layers.1.attn.q_proj.weight"].dtype == torch.bfloat16       # the run's storage rule, where no spec states a type
        seqs = {"a": [3, 14, 15, 9, 2, 6, 5, 35, 8, 9, 7, 9, 3, 2, 38, 4, 6, 1, 0, 22, 31], "b": [2, 7, 18, 28, 18, 2, 8, 4, 5, 9, 0, 12]}
        want = {r: latent_plain(weights, c, t) for r, t in seqs.items()}
        for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
            engine = Engine.load(folder, dtype=dtype, kv_tokens=64, page_tokens=4, max_requests=2)
            needs = engine.model.cache_needs()
            assert [len(n.tensors) for n in needs] == [1, 2, 1, 2] and len(engine.cache.groups) == 2
            assert engine._paged[0]["latent"].dtype == torch.float32 and tuple(engine._paged[0]["latent"].shape) == (2, 16, 4, c.latent)
            assert engine._paged[1]["k"].dtype == engine.act_dtype and tuple(engine._paged[1]["v"].shape) == (2, 16, 2, 8, 4)
            assert engine.model.blocks[0].mixer.gain.dtype == torch.float32
            every = lambda t: list(range(len(t)))
            whole = {}
            for r, t in seqs.items():
                engine.add_request(r)
                whole[r] = engine.step([StepEntry(r, t, every(t))]).clone()
                engine.end_request(r)
                assert (whole[r].cpu().double() - want[r]).abs().max() < tol * want[r].abs().max(), (dtype, r)
            # portions of one beside single tokens of the other, over page edges, pages of ended requests used again
            engine.add_request("a")
            engine.add_request("b")
            at, rows = {"a": 0, "b": 0}, {"a": [], "b": []}
            for na, nb in [(5, 1), (2, 1), (1, 3), (6, 1), (3, 2), (2, 4), (2, 0)]:
                entries = []
                for r, n in (("a", na), ("b", nb)):
                    n = min(n, len(seqs[r]) - at[r])
                    if n:
                        entries.append(StepEntry(r, seqs[r][at[r]:at[r] + n], list(range(n))))
                out = engine.step(entries)
                i = 0
                for e in entries:
                    rows[e.request].append(out[i:i + len(e.tokens)].clone())
                    i += len(e.tokens)
                    at[e.request] += len(e.tokens)
            for r in seqs:
                assert at[r] == len(seqs[r])
                got = torch.cat(rows[r])
                assert (got.cpu().double() - want[r]).abs().max() < tol * want[r].abs().max()
                if dtype == "float32":
                    assert (got - whole[r]).abs().max() < 1e-5 * whole[r].abs().max()
            engine.end_request("a")
            engine.end_request("b")
            assert engine.cache.pages_in_use(0) == 0 and engine.cache.pages_in_use(1) == 0
    finally:
        unregister_architecture("ToyLatentForCausalLM")
        unregister("mixer", "toy_latent")


@pytest.mark.parametrize("dtype,page", [("float32", 4), ("bfloat16", 16)])
def test_window_attention_gives_pages_back(dtype, page):
    """A second cache group: odd layers keep a window of 10 keys.  Their pages go back as the window passes, the logits
    equal the plain implementation with the same window, in portions as whole."""
    from helpers import TINY_A, model_folder, plain
    from llmx_amd import Engine, MiniMaxM3Config
    from llmx_amd.engine import StepEntry
    from llmx_amd.models import assemble
    from llmx_amd.weights import ModelFiles, load as load_weights
    W = 10
    cfg = MiniMaxM3Config(**TINY_A)
    spec = assemble(cfg)
    spec.blocks[1].mixer.params["window"] = W
    files = ModelFiles(model_folder("A"))
    exact = dtype == "float32"
    engine = Engine(cfg, spec, dtype, kv_tokens=160, page_tokens=page, max_requests=2,
                    weights=lambda e: load_weights(e.model.tensor_specs(set(files.names())), files, e.device, exact))
    assert [g.window for g in engine.cache.groups] == [None, W]
    config, w = plain("A")
    tokens = [(7 * i + 3) % 256 for i in range(70)]
    rt = None if exact else torch.bfloat16
    x = w["model.embed_tokens.weight"].double()[tokens]
    for i in range(2):
        p = f"model.layers.{i}."
        h = pm.rms_norm(x, w[p + "input_layernorm.weight"].double(), config["rms_norm_eps"])
        x = x + pm.attention_layer(h, list(range(70)), w, p + "self_attn.", config, rt, window=W if i == 1 else None)
        h = pm.rms_norm(x, w[p + "post_attention_layernorm.weight"].double(), config["rms_norm_eps"])
        x = x + pm.moe_layer(h, w, p + "mlp.", config, rt)[0]
    want = pm._rounded(pm.rms_norm(x, w["model.norm.weight"].double(), config["rms_norm_eps"]), rt) @ w["lm_head.weight"].double().T
    engine.add_request("p")
    rows, held = [], []
    for a, b in ((0, 13), (13, 15), (15, 40), (40, 41), (41, 42), (42, 70)):
        rows.append(engine.step([StepEntry("p", tokens[a:b], list(range(b - a)))]).clone())
        held.append((engine.cache.pages_held("p", 0), engine.cache.pages_held("p", 1)))
    got = torch.cat(rows).cpu().double()
    tol = 2e-5 if exact else 3e-2
    assert (got - want).abs().max() <= tol * want.abs().max()
    assert held[-1][0] == -(-70 // page) and held[-1][1] <= -(-W // page) + 1       # the window's group holds a window's worth
    if exact:
        engine.add_request("w")
        whole = engine.step([StepEntry("w", tokens, list(range(70)))])
        assert torch.equal(whole, torch.cat(rows))
        engine.end_request("w")
    engine.end_request("p")
    assert engine.cache.pages_in_use(0) == 0 and engine.cache.pages_in_use(1) == 0
    # told the most tokens a step brings of a request, the engine makes the window's pool for windows, not for contexts;
    # portions within the bound give the same logits through it
    small = Engine(cfg, spec, dtype, kv_tokens=160, page_tokens=page, max_requests=2, step_tokens=12,
                   weights=lambda e: load_weights(e.model.tensor_specs(set(files.names())), files, e.device, exact))
    pools = [g.n_pages for g in small.cache.groups]
    assert pools[0] == 160 // page and pools[1] == 2 * (-(-(W + 12) // page) + 1) < pools[0]
    assert small._paged[1]["k"].shape[1] == pools[1]
    small.add_request("q")
    small.add_request("other")
    cut = []
    for a in range(0, 70, 12):
        cut.append(small.step([StepEntry("q", tokens[a:a + 12], list(range(len(tokens[a:a + 12])))),
                               StepEntry("other", tokens[69 - a:69 - a + 1], [])])[:len(tokens[a:a + 12])].clone())
    assert (torch.cat(cut).cpu().double() - want).abs().max() <= tol * want.abs().max()
    if exact:
        assert torch.equal(torch.cat(cut), torch.cat(rows))
