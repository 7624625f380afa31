"""The plain implementation: MiniMax-M3 written straight from the reference's formulas.

Whole sequences, no cache, no batching, one function for each part, torch on the CPU used as a calculator (float64 by
default).  It shares no code with llmx_amd: it reads config.json with `json` and the weights with the `safetensors`
package.  Every function cites the lines of /root/reference it was written from.

`round_to=torch.bfloat16` rounds the inputs of weight products, the cached keys and values, and the attention output to
bfloat16 (and widens them again), the places where the serving path stores bfloat16; every sum, norm, softmax, rotation,
router logit and the residual stay in `dtype`.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# ---------------------------------------------------------------------------
def load_folder(folder):
    """(config dict, {name: tensor}) of a model folder, read without llmx_amd."""
    from safetensors import safe_open
    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name)
    return config, weights


def _rounded(x, round_to):
    return x if round_to is None else x.to(round_to).to(x.dtype)


# ---------------------------------------------------------------------------
def rms_norm(x, weight, eps):
    """y = x * (r * w), r = 1 / sqrt(mean(x^2) + eps); no mean subtraction, no bias.

    src/backends/cpu/cpu_backend.hpp:1437-1459 (rms_norm_raw): s = sum x^2; r = 1/sqrt(s/n + eps); dst = x * (r * w).
    """
    n = x.shape[-1]
    s = (x * x).sum(dim=-1, keepdim=True)
    r = 1.0 / torch.sqrt(s / n + eps)
    return x * (r * weight)


def rope_tables(positions, rotary_dim, theta):
    """cos, sin [len(positions), rotary_dim/2], float32 values in the reference's float32 arithmetic.

    src/model/rope.hpp:25-28 (reciprocal_power: 1.0f / powf(theta, 2.0f*i/dim)), :203-210 (cosf((float)pos * freq[i])).
    powf, cosf and sinf are taken as correctly rounded: evaluated in float64 on their float32 arguments and rounded once.
    """
    half = rotary_dim // 2
    i = torch.arange(half, dtype=torch.float32)
    exponent = 2.0 * i / float(rotary_dim)                                             # float32
    power = torch.pow(torch.tensor(theta, dtype=torch.float32).double(), exponent.double()).float()
    freq = 1.0 / power                                                                 # float32
    pos = torch.as_tensor(positions, dtype=torch.float32)[:, None]
    angle = (pos * freq[None, :]).double()                                             # the float32 product, widened
    return torch.cos(angle).float(), torch.sin(angle).float()


def apply_partial_rope(x, cos, sin, rotary_dim):
    """NeoX halves over the first rotary_dim values of each head; the rest pass through.

    x [T, H, D].  For i < R/2 with a = i, b = i + R/2: x'_a = x_a cos - x_b sin, x'_b = x_b cos + x_a sin.
    src/backends/cpu/cpu_backend.hpp:1461-1480 (rope_raw).
    """
    half = rotary_dim // 2
    if half == 0:
        return x
    c = cos.to(x.dtype)[:, None, :]
    s = sin.to(x.dtype)[:, None, :]
    a = x[..., :half]
    b = x[..., half:rotary_dim]
    out = x.clone()
    out[..., :half] = a * c - b * s
    out[..., half:rotary_dim] = b * c + a * s
    return out


def causal_attention(q, k, v, window=None):
    """Causal grouped-query softmax attention of one sequence.

    q [T, Hq, D], k and v [T, Hkv, D].  Row at position p, head h reads KV head h // (Hq // Hkv): score_j = q.k_j / sqrt(D)
    for j <= p (and j > p - window under a window); p_j = exp(score_j - max) / sum; out = sum_j p_j v_j.
    src/backends/cpu/cpu_backend.hpp:971-1104 (attention): scale 1/sqrt(head_dim) :984, kvh = h / ratio :1002,
    max then exp then sum :1005-1028, normalized before the value sum :1030, values summed in token order :1070-1099.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    ratio = Hq // Hkv
    scale = 1.0 / math.sqrt(D)
    out = torch.zeros_like(q)
    for h in range(Hq):
        kvh = h // ratio
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            scores = (k[lo:p + 1, kvh, :] @ q[p, h, :]) * scale
            w = torch.exp(scores - scores.max())
            w = w / w.sum()
            out[p, h, :] = w @ v[lo:p + 1, kvh, :]
    return out


def attention_layer(h, positions, w, prefix, cfg, round_to=None, window=None):
    """q, k, v projections; RMSNorm over the whole q and the whole k projection; partial rotary; attention; output projection.

    src/model/arch/minimax_m3.hpp:255-259,270-271 for the order (projections, norm + rotation on q and k, attention,
    output projection joined into the residual by the caller).  The norm here spans the whole projection (weight of
    width heads*head_dim) where the reference's module norms each head (weight of width head_dim): that is this
    architecture's variant; the formula of the norm itself is rms_norm above.
    """
    T = h.shape[0]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    dt = h.dtype
    hin = _rounded(h, round_to)
    q = hin @ w[prefix + "q_proj.weight"].to(dt).T
    k = hin @ w[prefix + "k_proj.weight"].to(dt).T
    v = hin @ w[prefix + "v_proj.weight"].to(dt).T
    q = rms_norm(q, w[prefix + "q_norm.weight"].to(dt), cfg["rms_norm_eps"])
    k = rms_norm(k, w[prefix + "k_norm.weight"].to(dt), cfg["rms_norm_eps"])
    R = rotary_dim_of(cfg)
    cos, sin = rope_tables(positions, R, theta_of(cfg))
    q = apply_partial_rope(q.view(T, Hq, D), cos, sin, R)
    k = apply_partial_rope(k.view(T, Hkv, D), cos, sin, R)
    q, k, v = _rounded(q, round_to), _rounded(k, round_to), _rounded(v.view(T, Hkv, D), round_to)
    o = _rounded(causal_attention(q, k, v, window).reshape(T, Hq * D), round_to)
    return o @ w[prefix + "o_proj.weight"].to(dt).T


def route(z, bias, k, normalize, scale):
    """Sigmoid scores, pick by score + bias (lowest id on ties), weights from the unbiased scores.

    src/backends/cpu/cpu_backend.hpp:2774-2819 (route_biased): s = 1/(1+exp(-z)) :2793; b = s + bias :2794; a row with a
    non-finite key gets no expert and zero weights :2797-2803; k picks of the largest b not yet taken, first found wins
    :2805-2813; divide = normalize and (sigmoid or k > 1) :2815; w_j = (divide ? s_j / sum : s_j) * scale :2817.
    Returns (ids [T, k] int64 with -1 for no expert, weights [T, k]).
    """
    T, X = z.shape
    s = 1.0 / (1.0 + torch.exp(-z))
    b = s + bias if bias is not None else s.clone()
    ids = torch.full((T, k), -1, dtype=torch.int64)
    weights = torch.zeros((T, k), dtype=z.dtype)
    for t in range(T):
        if not torch.isfinite(b[t]).all():
            continue
        taken = [False] * X
        chosen = []
        for j in range(k):
            best = -1
            for e in range(X):
                if not taken[e] and (best < 0 or b[t, e] > b[t, best]):
                    best = e
            taken[best] = True
            ids[t, j] = best
            chosen.append(s[t, best])
        total = sum(chosen)
        for j in range(k):
            weights[t, j] = (chosen[j] / total if normalize else chosen[j]) * scale
    return ids, weights


def swiglu_expert(h, gate_up, down, round_to=None):
    """One expert: a = silu(h.Wg^T) * (h.Wu^T); y = a.Wd^T.  gate_up holds the gate rows first.

    src/backends/cpu/cpu_backend.hpp:3003-3010 (swiglu, GluForm::silu, limit 0: silu_of(g) * u);
    gate rows first in the fused tensor: tests/fixture_minimax.py:153-155,177-190.
    """
    F = gate_up.shape[0] // 2
    g = h @ gate_up[:F].T
    u = h @ gate_up[F:].T
    a = (g / (1.0 + torch.exp(-g))) * u
    return _rounded(a, round_to) @ down.T


def forced_route(z, bias, picks, normalize, scale):
    """The weights route() gives when the picks are `picks` [T, k] instead of its own: for comparing a path that rounds
    to bfloat16, where a key within rounding of a tie may fall either way.  Same formulas as route()."""
    s = 1.0 / (1.0 + torch.exp(-z))
    chosen = torch.gather(s, 1, picks)
    if normalize:
        total = torch.zeros(z.shape[0], dtype=z.dtype)
        for j in range(picks.shape[1]):
            total = total + chosen[:, j]
        chosen = chosen / total[:, None]
    return picks, chosen * scale


def moe_layer(h, w, prefix, cfg, round_to=None, picks=None):
    """Router on the unrounded rows, experts on the rounded ones, results weighted and summed in slot order.

    Router logits always in full precision: src/backends/backend.hpp:944-947.  Combine: acc = sum_j w_j * y_j in slot
    order, a slot without an expert adds nothing: src/backends/cpu/cpu_backend.hpp:2840-2867.
    """
    dt = h.dtype
    z = h @ w[prefix + "gate.weight"].to(dt).T
    bias = w[prefix + "gate.e_score_correction_bias"].to(dt)
    if picks is None:
        ids, weights = route(z, bias, cfg["num_experts_per_tok"], cfg["norm_topk_prob"], cfg["routed_scaling_factor"])
    else:
        ids, weights = forced_route(z, bias, picks, cfg["norm_topk_prob"], cfg["routed_scaling_factor"])
    hin = _rounded(h, round_to)
    gate_up = w[prefix + "experts.gate_up_proj"]      # indexed by expert before widening: only the picked experts are touched
    down = w[prefix + "experts.down_proj"]
    # each picked expert's output for the rows that picked it (an expert's weights are widened once) ...
    y = torch.zeros(ids.shape[0], ids.shape[1], h.shape[1], dtype=dt)
    for e in sorted(set(ids.flatten().tolist()) - {-1}):
        rows, slots = torch.nonzero(ids == e, as_tuple=True)
        y[rows, slots] = swiglu_expert(hin[rows], gate_up[e].to(dt), down[e].to(dt), round_to)
    # ... and each row's weighted sum in slot order
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        acc = torch.zeros(h.shape[1], dtype=dt)
        for j in range(ids.shape[1]):
            if int(ids[t, j]) >= 0:
                acc = acc + weights[t, j] * y[t, j]
        out[t] = acc
    keys = 1.0 / (1.0 + torch.exp(-z)) + bias
    return out, ids, weights, keys, z


def rotary_dim_of(cfg):
    if "rotary_dim" in cfg:
        return cfg["rotary_dim"]
    return int(cfg["head_dim"] * cfg["rope_parameters"]["partial_rotary_factor"])


def theta_of(cfg):
    return cfg["rope_parameters"]["rope_theta"] if "rope_parameters" in cfg else cfg["rope_theta"]


def forward(cfg, w, tokens, dtype=torch.float64, round_to=None, return_routing=False, positions=None, picks=None):
    """Logits [T, vocab] of one whole sequence.

    Embedding (src/model/arch/blocks.hpp:95-97), per layer norm -> mixer joined -> norm -> experts joined
    (src/model/arch/minimax_m3.hpp:247-287, pre-norm, two residual adds), final norm and head (blocks.hpp:267-272).
    `picks` (per layer [T, k] expert ids) replaces the router's own picks; `return_routing` also returns per layer
    (ids, weights, keys, z) with the router logits z and keys = sigmoid(z) + bias.
    """
    tokens = list(tokens)
    T = len(tokens)
    positions = list(range(T)) if positions is None else list(positions)
    x = w["model.embed_tokens.weight"][tokens].to(dtype)
    eps = cfg["rms_norm_eps"]
    routing = []
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        h = rms_norm(x, w[p + "input_layernorm.weight"].to(dtype), eps)
        x = x + attention_layer(h, positions, w, p + "self_attn.", cfg, round_to)
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"].to(dtype), eps)
        y, ids, weights, keys, z = moe_layer(h, w, p + "mlp.", cfg, round_to, None if picks is None else picks[layer])
        routing.append((ids, weights, keys, z))
        x = x + y
    h = _rounded(rms_norm(x, w["model.norm.weight"].to(dtype), eps), round_to)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    logits = h @ head.to(dtype).T
    return (logits, routing) if return_routing else logits


def greedy(cfg, w, prompt, n_new, dtype=torch.float64, round_to=None):
    """n_new greedy tokens after the prompt, each from a whole forward pass; ties take the lowest id."""
    tokens = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, w, tokens, dtype, round_to)[-1]
        nxt = int(torch.argmax(logits))  # torch returns the first maximal index
        out.append(nxt)
        tokens.append(nxt)
    return out
