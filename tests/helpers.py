"""Shared by the tests: the two tiny configurations, model folders in a temporary place, and ways of cutting a run."""

from __future__ import annotations

import os
import random
import tempfile
from functools import lru_cache

import torch

import plain_model
from llmx_amd import MiniMaxM3Config, RandomInit
from llmx_amd.weights.folder import write_random_model

# The two tiny configurations differ in every size and option.
TINY_A = dict(vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              rotary_dim=8, rope_theta=1e4, rms_norm_eps=1e-6, num_local_experts=8, num_experts_per_tok=2, intermediate_size=32,
              routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False, max_position_embeddings=1024)
INIT_A = RandomInit(seed=0, std=0.02, norm_std=0.0, bias_range=0.0, storage="bfloat16")
PAGE_A = 4

TINY_B = dict(vocab_size=320, hidden_size=96, num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=1, head_dim=24,
              rotary_dim=24, rope_theta=1e6, rms_norm_eps=1e-5, num_local_experts=16, num_experts_per_tok=4, intermediate_size=48,
              routed_scaling_factor=2.5, norm_topk_prob=False, tie_word_embeddings=False, max_position_embeddings=2048)
INIT_B = RandomInit(seed=1, std=0.05, norm_std=0.1, bias_range=0.1, storage="bfloat16")
PAGE_B = 8

# "A16": configuration A on pages of 16 tokens, where bfloat16 attention runs on the matrix cores
TINY = {"A": (TINY_A, INIT_A, PAGE_A), "B": (TINY_B, INIT_B, PAGE_B), "A16": (TINY_A, INIT_A, 16)}

_TMP = tempfile.TemporaryDirectory(prefix="llmx_amd_tests_")


@lru_cache(maxsize=None)
def model_folder(name: str) -> str:
    """A model folder of tiny configuration `name`, written once per test run into a temporary folder."""
    cfg, init, _ = TINY[name]
    folder = os.path.join(_TMP.name, f"tiny_{name}")
    write_random_model(folder, MiniMaxM3Config(**cfg), init)
    return folder


@lru_cache(maxsize=None)
def plain(name: str):
    """(config dict, weights) of the folder as the plain implementation reads them."""
    return plain_model.load_folder(model_folder(name))


def tokens_for(name: str, length: int, seed: int):
    rng = random.Random(1000 * seed + length)
    vocab = TINY[name][0]["vocab_size"]
    return [rng.randrange(vocab) for _ in range(length)]


@lru_cache(maxsize=None)
def plain_logits(name: str, length: int, seed: int, rounded: bool):
    cfg, w = plain(name)
    return plain_model.forward(cfg, w, tokens_for(name, length, seed), torch.float64,
                               torch.bfloat16 if rounded else None)


def routing_margin(name: str, tokens, rounded: bool = False) -> float:
    """Smallest gap, over all rows and layers, between the last pick's key and the best key left out."""
    cfg, w = plain(name)
    _, routing = plain_model.forward(cfg, w, tokens, torch.float64, torch.bfloat16 if rounded else None, return_routing=True)
    k = cfg["num_experts_per_tok"]
    margin = float("inf")
    for _, _, keys, _ in routing:
        top = torch.sort(keys, dim=-1, descending=True).values
        margin = min(margin, float((top[:, k - 1] - top[:, k]).min()))
    return margin


@lru_cache(maxsize=None)
def row_margins(name: str, length: int, seed: int, rounded: bool):
    """Per row, the smallest gap over the layers between the last pick's key and the best key left out."""
    cfg, w = plain(name)
    _, routing = plain_model.forward(cfg, w, tokens_for(name, length, seed), torch.float64, torch.bfloat16 if rounded else None,
                                     return_routing=True)
    k = cfg["num_experts_per_tok"]
    margins = torch.full((length,), float("inf"), dtype=torch.float64)
    for _, _, keys, _ in routing:
        top = torch.sort(keys, dim=-1, descending=True).values
        margins = torch.minimum(margins, top[:, k - 1] - top[:, k])
    return margins


class RoutingRecorder:
    """An engine observer that keeps every routed layer's picks and router logits by (request, position)."""

    def __init__(self, n_layers):
        self.n_layers = n_layers
        self.picks = {}    # request -> {position: [ids per layer]}
        self.logits = {}   # request -> {position: [router logits per layer]}

    def __call__(self, step, kind, **tensors):
        if kind != "routing":
            return
        ids = tensors["ids"].cpu()
        z = tensors["logits"].cpu()
        for e in step.entries:
            rows = self.picks.setdefault(e.request, {})
            zrows = self.logits.setdefault(e.request, {})
            for r in range(e.n):
                rows.setdefault(e.past + r, [None] * self.n_layers)[step.run_index] = ids[e.row0 + r].long()
                zrows.setdefault(e.past + r, [None] * self.n_layers)[step.run_index] = z[e.row0 + r].clone()

    def of(self, request, length):
        """Per layer [length, k] picks of a request."""
        rows = self.picks[request]
        return [torch.stack([rows[p][layer] for p in range(length)]) for layer in range(self.n_layers)]

    def logits_of(self, request, length):
        """Per layer [length, experts] float32 router logits of a request, as the engine computed them."""
        rows = self.logits[request]
        return [torch.stack([rows[p][layer] for p in range(length)]) for layer in range(self.n_layers)]


# A pick must be one of the k best keys of the engine's OWN router logits.  Keys are float32 values of about 1; the
# kernel's expf and the host's differ in the last place, so a key may lie below the k-th best by a few units of 6e-8.
PICK_SLACK = 4e-7
# The engine's router logits against the plain implementation's (run with the engine's picks in the layers before),
# relative to the largest logit (at least 1).  float32: sums of float32 products in another order; the largest
# difference met over all configurations of these tests is 2.5e-6.  bfloat16: the router reads unrounded rows in both;
# what differs lies upstream: the engine rounds the softmax weights to bfloat16 as the value product's operand, which
# the plain implementation does not, and single roundings fall the other way; the largest difference met is 6.0e-3
# (the test session prints what it met).
ROUTER_TOL = {False: 1e-5, True: 1e-2}
MEASURED = {"pick_gap": 0.0, "router_f32": 0.0, "router_bf16": 0.0}


def plain_logits_with_picks(name, tokens, picks, rounded=True, engine_logits=None):
    """The plain implementation's logits under the engine's expert picks, after checking every row's picks: no expert
    twice, and each pick's key (sigmoid of the engine's own router logit in float32, plus the bias) among the k best
    of that row within PICK_SLACK; the engine's router logits lie within ROUTER_TOL of the plain ones."""
    cfg, w = plain(name)
    logits, routing = plain_model.forward(cfg, w, tokens, torch.float64, torch.bfloat16 if rounded else None,
                                          return_routing=True, picks=picks)
    k = cfg["num_experts_per_tok"]
    for layer, (ids, _, keys, z) in enumerate(routing):
        assert all(len(set(row.tolist())) == k for row in ids), f"layer {layer}: an expert was picked twice"
        if engine_logits is None:
            own = keys
            slack = 1e-5
        else:
            ze = engine_logits[layer].float()
            bias = w[f"model.layers.{layer}.mlp.gate.e_score_correction_bias"].float()
            own = (1.0 / (1.0 + torch.exp(-ze)) + bias).double()
            slack = PICK_SLACK
            scale = max(1.0, float(z.abs().max()))
            gap = float((ze.double() - z).abs().max()) / scale
            MEASURED["router_bf16" if rounded else "router_f32"] = max(MEASURED["router_bf16" if rounded else "router_f32"], gap)
            assert gap <= ROUTER_TOL[rounded], f"layer {layer}: the engine's router logits differ from the plain ones by {gap:.3e} of the largest"
        kth = torch.sort(own, dim=-1, descending=True).values[:, k - 1]
        chosen = torch.gather(own, 1, ids)
        MEASURED["pick_gap"] = max(MEASURED["pick_gap"], float((kth[:, None] - chosen).max()))
        assert (chosen >= kth[:, None] - slack).all(), f"layer {layer}: the engine picked an expert whose key is not among the best {k}"
    return logits


def portions(total: int, sizes=(7, 2, 13, 3, 64, 2, 5, 31, 2, 17)):
    """Cuts [0, total) into portions of changing size, down to two tokens."""
    cuts, at, i = [], 0, 0
    while at < total:
        n = min(sizes[i % len(sizes)], total - at)
        cuts.append((at, at + n))
        at += n
        i += 1
    return cuts
