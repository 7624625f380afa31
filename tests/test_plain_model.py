"""What fixes the plain implementation beside the reference's text: special cases that reduce to a library routine,
invariants, and vectors the reference's own tests hold.  Each is chosen so that a plausible mistake (a wrong sign or
pairing, a norm in the wrong place, the wrong head mapping, halves swapped) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm
from helpers import TINY_A, TINY_B, plain, tokens_for

torch.manual_seed(0)
D64 = torch.float64


def rand(*shape):
    return torch.randn(*shape, dtype=D64)


# -- RMSNorm -------------------------------------------------------------------
def test_rms_norm():
    x, w = rand(5, 48) * 3, 1 + 0.1 * rand(48)
    lib = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), lib, rtol=1e-12)
    unit = pm.rms_norm(x, torch.ones(48, dtype=D64), 0.0)
    assert torch.allclose(unit.pow(2).mean(-1), torch.ones(5, dtype=D64))            # w = 1, eps = 0: the output's RMS is 1
    assert torch.allclose(pm.rms_norm(7.5 * x, w, 0.0), pm.rms_norm(x, w, 0.0))       # scale invariant without eps
    assert torch.equal(pm.rms_norm(torch.zeros(2, 48, dtype=D64), w, 1e-6), torch.zeros(2, 48, dtype=D64))   # not NaN
    assert not torch.allclose(pm.rms_norm(x * 1e-3, w, 1e-5), pm.rms_norm(x * 1e-3, w, 1e-6))                # eps is read
    assert not torch.allclose(pm.rms_norm(x, w, 0.0).mean(-1), torch.zeros(5, dtype=D64), atol=1e-3)        # no mean subtraction


def test_norm_over_the_whole_projection_couples_the_heads():
    """With one head it is the per-head norm; with several, scaling one head's values changes the others' outputs."""
    x, w = rand(3, 4 * 16), torch.ones(64, dtype=D64)
    whole = pm.rms_norm(x, w, 1e-6).view(3, 4, 16)
    per_head = pm.rms_norm(x.view(3, 4, 16), torch.ones(16, dtype=D64), 1e-6)
    assert not torch.allclose(whole, per_head)
    one = rand(3, 16)
    assert torch.allclose(pm.rms_norm(one, torch.ones(16, dtype=D64), 1e-6), pm.rms_norm(one.view(3, 1, 16), torch.ones(16, dtype=D64), 1e-6).view(3, 16))
    x2 = x.clone()
    x2[:, :16] *= 10.0
    assert not torch.allclose(pm.rms_norm(x2, w, 1e-6)[:, 16:], pm.rms_norm(x, w, 1e-6)[:, 16:])


# -- rotary ----------------------------------------------------------------------
@pytest.mark.parametrize("D,R,theta", [(16, 8, 1e4), (24, 24, 1e6), (128, 64, 5e6)])
def test_rope(D, R, theta):
    T, H = 9, 3
    pos = [0, 1, 2, 5, 17, 100, 1000, 4095, 65535]
    cos, sin = pm.rope_tables(pos, R, theta)
    # the tables against a loop in float32 arithmetic (the reference fills them so: rope.hpp:203-210), float32 roundings made with struct
    import struct
    f32 = lambda v: struct.unpack("f", struct.pack("f", v))[0]
    for pi, p in enumerate(pos):
        for i in range(R // 2):
            freq = f32(1.0 / f32(math.pow(f32(theta), f32(f32(2.0 * i) / R))))
            angle = f32(float(p) * freq)
            assert float(cos[pi, i]) == f32(math.cos(angle)) and float(sin[pi, i]) == f32(math.sin(angle))
    x = rand(T, H, D)
    y = pm.apply_partial_rope(x, cos, sin, R)
    assert torch.equal(y[0], x[0])                                       # position 0 is the identity
    assert torch.equal(y[..., R:], x[..., R:])                           # dims [R, D) pass through untouched
    half = R // 2
    # a complex multiply on the pairs (i, i + R/2): (a + ib) * (cos + i sin)
    z = torch.complex(x[..., :half], x[..., half:R]) * torch.complex(cos.double(), sin.double())[:, None, :]
    assert torch.allclose(y[..., :half], z.real) and torch.allclose(y[..., half:R], z.imag)
    assert torch.allclose(y[..., :half] ** 2 + y[..., half:R] ** 2, x[..., :half] ** 2 + x[..., half:R] ** 2)   # each pair's norm is kept
    # interleaved pairing (i, i+1) would differ
    if R >= 4:
        zi = torch.view_as_complex(x[..., :R].reshape(T, H, half, 2).contiguous()) * torch.complex(cos.double(), sin.double())[:, None, :]
        assert not torch.allclose(y[..., :R], torch.view_as_real(zi).reshape(T, H, R))
    # only distances count: <rope(q, m), rope(k, n)> = <rope(q, m + s), rope(k, n + s)>
    q, k = rand(1, 1, D), rand(1, 1, D)
    def dot(m, n):
        cm, sm = pm.rope_tables([m], R, theta)
        cn, sn = pm.rope_tables([n], R, theta)
        return float((pm.apply_partial_rope(q, cm, sm, R) * pm.apply_partial_rope(k, cn, sn, R)).sum())
    assert abs(dot(7, 3) - dot(107, 103)) < 1e-4 * (1 + abs(dot(7, 3)))
    assert abs(dot(7, 3) - dot(3, 7)) > 1e-6                              # and their sign: swapping the positions changes it


# -- attention ---------------------------------------------------------------------
@pytest.mark.parametrize("Hq,Hkv,D", [(4, 2, 16), (8, 1, 24), (6, 6, 32)])
def test_attention_against_library(Hq, Hkv, D):
    T = 13
    q, k, v = rand(T, Hq, D), rand(T, Hkv, D), rand(T, Hkv, D)
    got = pm.causal_attention(q, k, v)
    rep = Hq // Hkv
    kk, vv = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)      # KV head of head h is h // rep
    scores = torch.einsum("thd,shd->hts", q, kk) / math.sqrt(D)
    scores = scores.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    lib = torch.einsum("hts,shd->thd", torch.softmax(scores, -1), vv)
    assert torch.allclose(got, lib, rtol=1e-10, atol=1e-12)
    lib2 = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(got, lib2, rtol=1e-8, atol=1e-10)
    assert torch.allclose(got[0], v[0].repeat_interleave(rep, dim=0))              # one key: the output is its value
    zero_q = pm.causal_attention(torch.zeros_like(q), k, v)
    assert torch.allclose(zero_q[4], vv[:5].mean(0))                               # q = 0: the mean of the values so far
    k2, v2 = k.clone(), v.clone()
    k2[8:], v2[8:] = rand(T - 8, Hkv, D), rand(T - 8, Hkv, D)
    assert torch.equal(pm.causal_attention(q, k2, v2)[:8], got[:8])                # later tokens never change earlier rows
    # a window of w keys: rows below w are as before, row p reads keys p-w+1 .. p
    win = pm.causal_attention(q, k, v, window=4)
    assert torch.equal(win[:4], got[:4]) and not torch.allclose(win[9], got[9])
    sc = torch.einsum("hd,shd->hs", q[9], kk[6:10]) / math.sqrt(D)
    assert torch.allclose(win[9], torch.einsum("hs,shd->hd", torch.softmax(sc, -1), vv[6:10]))


def test_attention_head_mapping():
    """Each KV head holds a constant value: the output of head h names the KV head it read (h // ratio, not h % kv_heads)."""
    T, Hq, Hkv, D = 5, 6, 3, 8
    v = torch.arange(Hkv, dtype=D64).view(1, Hkv, 1).expand(T, Hkv, D).contiguous()
    out = pm.causal_attention(rand(T, Hq, D), rand(T, Hkv, D), v)
    assert torch.allclose(out[:, :, 0], torch.tensor([0, 0, 1, 1, 2, 2], dtype=D64).expand(T, Hq))


# -- router ----------------------------------------------------------------------
def test_route():
    T, X, k = 11, 24, 5
    z, bias = rand(T, X) * 2, rand(X) * 0.3
    ids, w = pm.route(z, bias, k, True, 2.5)
    s = torch.sigmoid(z)
    top = torch.topk(s + bias, k, dim=-1)                                 # library top-k, best first
    assert torch.equal(ids, top.indices)
    chosen = torch.gather(s, 1, ids)
    assert torch.allclose(w, chosen / chosen.sum(-1, keepdim=True) * 2.5)
    assert torch.allclose(w.sum(-1), torch.full((T,), 2.5, dtype=D64))    # normalized weights sum to the scale
    ids_u, w_u = pm.route(z, bias, k, False, 2.5)
    assert torch.equal(ids_u, ids) and torch.allclose(w_u, chosen * 2.5)  # un-normalized: the unbiased scores times the scale
    ids_c, w_c = pm.route(z, bias + 0.7, k, True, 2.5)
    assert torch.equal(ids_c, ids) and torch.allclose(w_c, w)             # one constant on every bias changes nothing
    big = bias.clone()
    big[3] = 50.0
    ids_b, w_b = pm.route(z, big, k, False, 1.0)
    assert (ids_b[:, 0] == 3).all() and torch.allclose(w_b[:, 0], s[:, 3])   # forced in by its bias, weighted by its score
    _, w1 = pm.route(z, bias, 1, True, 2.5)
    assert torch.equal(w1, torch.full((T, 1), 2.5, dtype=D64))            # k = 1 normalized: the weight is the scale
    # ties take the lowest id; a non-finite key gives no expert and zero weights (cpu_backend.hpp:2797-2813)
    zt = torch.zeros(2, 6, dtype=D64)
    zt[1, 2] = float("nan")
    ids_t, w_t = pm.route(zt, None, 3, True, 1.0)
    assert ids_t[0].tolist() == [0, 1, 2] and ids_t[1].tolist() == [-1, -1, -1] and w_t[1].tolist() == [0, 0, 0]
    zi = torch.zeros(1, 4, dtype=D64)
    zi[0, 1], zi[0, 2] = float("inf"), float("-inf")                      # sigmoid gives 1 and 0: finite keys
    assert pm.route(zi, None, 2, False, 1.0)[0].tolist() == [[1, 0]]


# -- experts ---------------------------------------------------------------------
def one_layer_weights(X, E, Fe, same=False):
    w = {"gate.weight": rand(X, E), "gate.e_score_correction_bias": rand(X) * 0.1,
         "experts.gate_up_proj": rand(X, 2 * Fe, E) * 0.3, "experts.down_proj": rand(X, E, Fe) * 0.3}
    if same:
        w["experts.gate_up_proj"][:] = w["experts.gate_up_proj"][0]
        w["experts.down_proj"][:] = w["experts.down_proj"][0]
    return w


def test_experts():
    E, Fe = 20, 12
    h = rand(7, E)
    cfg = dict(num_experts_per_tok=1, norm_topk_prob=True, routed_scaling_factor=1.7)
    w = one_layer_weights(1, E, Fe)
    out, ids, weights, _, _ = pm.moe_layer(h, w, "", cfg)
    gu, dn = w["experts.gate_up_proj"][0], w["experts.down_proj"][0]
    mlp = (F.silu(h @ gu[:Fe].T) * (h @ gu[Fe:].T)) @ dn.T                 # one expert, one pick: a plain SwiGLU MLP times the scale
    assert torch.allclose(out, 1.7 * mlp, rtol=1e-10)
    swapped = dict(w)
    swapped["experts.gate_up_proj"] = torch.cat([gu[Fe:], gu[:Fe]])[None]
    assert not torch.allclose(pm.moe_layer(h, swapped, "", cfg)[0], out)   # gate rows come first
    # identical experts, normalized weights: the output does not depend on the routing
    cfg3 = dict(num_experts_per_tok=3, norm_topk_prob=True, routed_scaling_factor=1.0)
    same = one_layer_weights(6, E, Fe, same=True)
    out_same = pm.moe_layer(h, same, "", cfg3)[0]
    gu, dn = same["experts.gate_up_proj"][0], same["experts.down_proj"][0]
    assert torch.allclose(out_same, (F.silu(h @ gu[:Fe].T) * (h @ gu[Fe:].T)) @ dn.T, rtol=1e-9)
    zero = one_layer_weights(6, E, Fe)
    zero["experts.down_proj"].zero_()
    assert torch.equal(pm.moe_layer(h, zero, "", cfg3)[0], torch.zeros(7, E, dtype=D64))   # no down projection: nothing is added
    # combine in slot order with the router's weights
    w6 = one_layer_weights(6, E, Fe)
    out6, ids6, weights6, _, _ = pm.moe_layer(h, w6, "", cfg3)
    t = 2
    want = sum(weights6[t, j] * pm.swiglu_expert(h[t], w6["experts.gate_up_proj"][ids6[t, j]], w6["experts.down_proj"][ids6[t, j]]) for j in range(3))
    assert torch.allclose(out6[t], want)


# -- whole model -------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_model_invariants(name):
    cfg, w = plain(name)
    tokens = tokens_for(name, 12, 3)
    logits = pm.forward(cfg, w, tokens)
    assert logits.shape == (12, cfg["vocab_size"]) and torch.isfinite(logits).all()
    # later tokens never change earlier logits
    other = tokens[:8] + tokens_for(name, 4, 9)
    assert torch.allclose(pm.forward(cfg, w, other)[:8], logits[:8], rtol=0, atol=1e-12)
    # a shift of all positions changes nothing: only distances count (tables are float32, hence the bound)
    shifted = pm.forward(cfg, w, tokens, positions=range(100, 112))
    assert (shifted - logits).abs().max() < 5e-5 * logits.abs().max()
    # without attention output and expert output the logits are head(norm(embed(id))), whatever the position or history
    w0 = dict(w)
    for key in w:
        if key.endswith("o_proj.weight") or key.endswith("experts.down_proj"):
            w0[key] = torch.zeros_like(w[key])
    bare = pm.forward(cfg, w0, tokens)
    x = w["model.embed_tokens.weight"].double()[tokens]
    want = pm.rms_norm(x, w["model.norm.weight"].double(), cfg["rms_norm_eps"]) @ w["lm_head.weight"].double().T
    assert torch.allclose(bare, want, rtol=1e-10)
    assert torch.allclose(pm.forward(cfg, w0, list(reversed(tokens))).flip(0), want, rtol=1e-10)


def test_greedy_and_rounding():
    cfg, w = plain("A")
    out = pm.greedy(cfg, w, [5, 17, 3], 4)
    assert len(out) == 4 and all(0 <= t < cfg["vocab_size"] for t in out)
    logits = pm.forward(cfg, w, [5, 17, 3])
    assert out[0] == int(logits[-1].argmax())
    # bfloat16 rounding: to nearest, ties to even, NaN stays NaN (core/bf16.hpp:5-11)
    x = torch.tensor([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, float("nan")], dtype=D64)
    r = pm._rounded(x, torch.bfloat16)
    assert r[0] == 1.0 and r[1] == 1.0 + 2.0 ** -6 and r[2] == 1.0 + 2.0 ** -7 and torch.isnan(r[3])
    rounded = pm.forward(cfg, w, [5, 17, 3, 9], round_to=torch.bfloat16)
    full = pm.forward(cfg, w, [5, 17, 3, 9])
    assert 0 < (rounded - full).abs().max() < 2e-2 * full.abs().max()


# -- points of the reading that no library routine fixes: each as an invariant a wrong reading breaks -----------------
def _attention_cfg():
    return dict(num_attention_heads=4, num_key_value_heads=2, head_dim=8, rotary_dim=4, rms_norm_eps=1e-6,
                rope_parameters={"rope_theta": 1e4})


def _attention_weights(scale=1.0):
    E, Hq, Hkv, D = 24, 4, 2, 8
    return {"q_proj.weight": rand(Hq * D, E) * scale, "k_proj.weight": rand(Hkv * D, E) * scale, "v_proj.weight": rand(Hkv * D, E) * scale,
            "o_proj.weight": rand(E, Hq * D) * scale, "q_norm.weight": 1 + 0.1 * rand(Hq * D), "k_norm.weight": 1 + 0.1 * rand(Hkv * D)}


def test_queries_and_keys_are_normed_and_values_are_not():
    """The norm (with the rotation) is applied to the q and k rows only; v goes to the cache as projected
    (/root/reference/src/model/arch/minimax_m3.hpp:258-259 norm q and k, :264 writes v_rows untouched).  A norm's output
    does not change when its input is scaled, so scaling W_q or W_k changes nothing (up to eps), while the output is
    linear in W_v: scaling W_v by c scales it by c, and W_v = 0 gives exactly 0.  Norming v as well, or forgetting the
    norm of q or k, breaks one of the three."""
    cfg, w = _attention_cfg(), _attention_weights()
    h = rand(6, 24)
    out = pm.attention_layer(h, list(range(6)), w, "", cfg)
    for name in ("q_proj.weight", "k_proj.weight"):
        scaled = dict(w)
        scaled[name] = w[name] * 7.0
        assert torch.allclose(pm.attention_layer(h, list(range(6)), scaled, "", cfg), out, rtol=1e-5, atol=1e-9), name
    scaled = dict(w)
    scaled["v_proj.weight"] = w["v_proj.weight"] * 7.0
    assert torch.allclose(pm.attention_layer(h, list(range(6)), scaled, "", cfg), 7.0 * out, rtol=1e-12)
    zero = dict(w)
    zero["v_proj.weight"] = torch.zeros_like(w["v_proj.weight"])
    assert torch.equal(pm.attention_layer(h, list(range(6)), zero, "", cfg), torch.zeros(6, 24, dtype=D64))
    # the norm comes before the rotation and spans the projection: a norm weight that differs inside a rotated pair is seen
    skew = dict(w)
    skew["q_norm.weight"] = w["q_norm.weight"].clone()
    skew["q_norm.weight"][0] *= 3.0
    assert not torch.allclose(pm.attention_layer(h, list(range(6)), skew, "", cfg), out)


def _bf16_by_hand(v: float) -> float:
    """Round to nearest, ties to even, on the bits (/root/reference/src/core/bf16.hpp:5-11), without torch's conversion."""
    import struct
    u = struct.unpack("<I", struct.pack("<f", v))[0]
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("<f", struct.pack("<I", u))[0]


def test_where_the_bfloat16_path_rounds():
    """The bfloat16 path rounds the inputs of weight products and what the cache stores, nothing else: sums, norms, the
    softmax, the router's logits and the residual stay wide (/root/reference/src/backends/backend.hpp:943-962: the
    router's product is F32 whatever the step's dtype, the experts' three products read their inputs in the step's dtype
    and sum in F32).  Each site is fixed by a vector whose rounding is worked out by hand on the bits."""
    bf = torch.bfloat16
    # the expert's activation is rounded once, before the down product; the sums are not rounded
    h = torch.tensor([3.0], dtype=D64)                       # exact in bfloat16: the caller has rounded it
    one = torch.ones(1, 1, dtype=D64)
    a = (3.0 / (1.0 + math.exp(-3.0))) * 3.0                 # silu(3) * 3 = 8.5731...
    y = pm.swiglu_expert(h, torch.cat([one, one]), one * 1.5, bf)
    assert float(y) == _bf16_by_hand(a) * 1.5 and float(y) != a * 1.5
    assert float(pm.swiglu_expert(h, torch.cat([one, one]), one * 1.5)) == pytest.approx(a * 1.5, rel=1e-15)
    # the layer rounds the rows the experts read and leaves the rows the router reads: a change below half a unit of
    # bfloat16's last place moves the router's logits and keys, and leaves every expert's output bit for bit
    E, X, Fi = 16, 4, 8
    cfg = dict(num_experts_per_tok=2, norm_topk_prob=False, routed_scaling_factor=1.0)
    w = {"gate.weight": rand(X, E), "gate.e_score_correction_bias": torch.zeros(X, dtype=D64),
         "experts.gate_up_proj": rand(X, 2 * Fi, E), "experts.down_proj": rand(X, E, Fi)}
    h = pm._rounded(rand(5, E), bf)
    nudged = h * (1.0 + 2.0 ** -11)                          # a quarter of a unit in the last place: rounds back to h
    assert torch.equal(pm._rounded(nudged, bf), h)
    base = pm.moe_layer(h, w, "", cfg, bf)
    moved = pm.moe_layer(nudged, w, "", cfg, bf, picks=base[1])
    assert not torch.equal(moved[4], base[4]) and torch.allclose(moved[4], base[4] * (1.0 + 2.0 ** -11), rtol=1e-12)   # the router saw it
    same_weights = pm.moe_layer(nudged, {**w, "gate.weight": torch.zeros(X, E, dtype=D64)}, "", cfg, bf, picks=base[1])[0]
    flat = pm.moe_layer(h, {**w, "gate.weight": torch.zeros(X, E, dtype=D64)}, "", cfg, bf, picks=base[1])[0]
    assert torch.equal(same_weights, flat)                   # with equal weights the experts' sum is the same bits: they read rounded rows
    # attention: the projections read rounded rows (a nudge below rounding changes nothing at all), and q, k, v and the
    # attention output are rounded where they are stored, so the layer's result differs from the wide one
    acfg, aw = _attention_cfg(), {k: pm._rounded(v, bf) for k, v in _attention_weights(0.3).items()}
    h = pm._rounded(rand(4, 24), bf)
    assert torch.equal(pm.attention_layer(h * (1.0 + 2.0 ** -11), [0, 1, 2, 3], aw, "", acfg, bf), pm.attention_layer(h, [0, 1, 2, 3], aw, "", acfg, bf))
    assert not torch.equal(pm.attention_layer(h * (1.0 + 2.0 ** -11), [0, 1, 2, 3], aw, "", acfg), pm.attention_layer(h, [0, 1, 2, 3], aw, "", acfg))
    # one key: the softmax weight is 1 and the layer's output is o_proj applied to the rounded v row, rounded again as
    # the attention output: worked out by hand for one element
    one_row = pm.attention_layer(h[:1], [0], aw, "", acfg, bf)
    v_row = [_bf16_by_hand(float(x)) for x in (h[:1] @ aw["v_proj.weight"].T)[0]]
    heads_v = torch.tensor([v_row[8 * (hq // 2) + d] for hq in range(4) for d in range(8)], dtype=D64)   # head hq reads KV head hq // 2
    assert torch.allclose(one_row[0], heads_v @ aw["o_proj.weight"].T, rtol=1e-12)
    # the whole model: the final norm's rows are rounded before the head, the residual never is
    cfg_a, w_a = plain("A")
    tokens = [5, 17, 3]
    x = w_a["model.embed_tokens.weight"].double()[tokens]
    w0 = {k: (torch.zeros_like(v) if k.endswith("o_proj.weight") or k.endswith("experts.down_proj") else v) for k, v in w_a.items()}
    rows = pm.rms_norm(x, w_a["model.norm.weight"].double(), cfg_a["rms_norm_eps"])
    want = torch.tensor([[_bf16_by_hand(float(v)) for v in r] for r in rows], dtype=D64) @ w_a["lm_head.weight"].double().T
    assert torch.allclose(pm.forward(cfg_a, w0, tokens, round_to=bf), want, rtol=1e-12)
