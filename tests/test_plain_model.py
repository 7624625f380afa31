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
    out, ids, weights, _ = pm.moe_layer(h, w, "", cfg)
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
    out6, ids6, weights6, _ = pm.moe_layer(h, w6, "", cfg3)
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
    assert torch.allclose(pm.forward(cfg, w0, tokens[::-1])[::-1] if False else pm.forward(cfg, w0, list(reversed(tokens))).flip(0), want, rtol=1e-10)


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
