"""Feed-forward parts: routed SwiGLU experts behind a scored top-k router, and a dense SwiGLU.

Router: z = h.Wr^T in float32 on unrounded rows (/root/reference/src/backends/backend.hpp:944-947); score sigmoid(z);
the pick key is score + correction bias, k picks, the lowest id on ties; weight = the unbiased score, divided by the
picks' sum when normalizing, times the scale (/root/reference/src/backends/cpu/cpu_backend.hpp:2774-2819).
Experts: a = silu(h.Wg_e^T) * (h.Wu_e^T), y = a.Wd_e^T (:3003-3010); the row's result is sum_j w_j * y_j in slot order
(:2840-2867).  The fused gate_up tensor holds gate rows first (/root/reference/tests/fixture_minimax.py:153-155).
"""

from __future__ import annotations

import re

import torch

from .. import ops
from ..limits import MAX_EXPERTS, MAX_TOP_K
from .base import FeedForward, register
from .spec import TensorSpec

_SCORES = {"sigmoid": ops.SCORE_SIGMOID, "softmax": ops.SCORE_SOFTMAX}


class RoutedExperts(FeedForward):
    """params: hidden, experts, top_k, intermediate, score ("sigmoid" | "softmax"), correction_bias (bool), normalize (bool), scale."""
    graph_safe = True

    wants_f32_input = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden = int(p["hidden"])
        self.experts = int(p["experts"])
        self.top_k = int(p["top_k"])
        self.intermediate = int(p["intermediate"])
        if p.get("score", "sigmoid") not in _SCORES:
            raise ValueError(f"router score {p.get('score')!r} is not one of {sorted(_SCORES)}")
        self.score = _SCORES[p.get("score", "sigmoid")]
        self.use_bias = bool(p.get("correction_bias", False))
        self.normalize = bool(p.get("normalize", True))
        self.scale = float(p.get("scale", 1.0))
        if not 0 < self.top_k <= self.experts:
            raise ValueError("experts per token must be between 1 and the expert count")
        if self.experts > MAX_EXPERTS or self.top_k > MAX_TOP_K:
            raise ValueError(f"routed experts: {self.experts} experts with {self.top_k} picks a token; the routing kernels take at most "
                             f"{MAX_EXPERTS} experts and {MAX_TOP_K} picks")
        self.per_expert = False
        self.w_router = self.bias = self.w_gate_up = self.w_down = None

    def tensor_specs(self, available):
        X, F, E = self.experts, self.intermediate, self.hidden
        specs = [TensorSpec(self.name("gate.weight"), (X, E), "router")]
        if self.use_bias:
            specs.append(TensorSpec(self.name("gate.e_score_correction_bias"), (X,), "bias"))
        fused = self.name("experts.gate_up_proj")
        single = re.compile(re.escape(self.name("experts.")) + r"\d+\.")
        has_single = any(single.match(n) for n in available)
        if has_single and fused in available:
            raise ValueError(f"{self.prefix}experts holds both fused and per-expert tensors")
        self.per_expert = has_single
        if has_single:
            # each expert's tensors go from the host straight into their places in the fused tensors
            down = self.name("experts.down_proj")
            for e in range(X):
                specs += [TensorSpec(self.name(f"experts.{e}.gate_proj.weight"), (F, E), into=(fused, (X, 2 * F, E), (e, slice(0, F)))),
                          TensorSpec(self.name(f"experts.{e}.up_proj.weight"), (F, E), into=(fused, (X, 2 * F, E), (e, slice(F, 2 * F)))),
                          TensorSpec(self.name(f"experts.{e}.down_proj.weight"), (E, F), into=(down, (X, E, F), (e,)))]
        else:
            specs += [TensorSpec(fused, (X, 2 * F, E)), TensorSpec(self.name("experts.down_proj"), (X, E, F))]
        return specs

    def load(self, tensors):
        self.w_router = tensors[self.name("gate.weight")]
        if self.use_bias:
            self.bias = tensors[self.name("gate.e_score_correction_bias")]
        # per-expert files arrive fused too (see tensor_specs)
        self.w_gate_up = tensors[self.name("experts.gate_up_proj")]
        self.w_down = tensors[self.name("experts.down_proj")]

    def takes_deferred_norm(self, step):
        return (ops.gemm_takes_normed_rows(step.rows, self.w_gate_up, step.act_dtype, ops.EPI_SWIGLU, grouped=True)
                and ops.gemm_f32_takes_normed_rows(step.rows, self.w_router))

    def forward(self, step, h, out, accumulate, h32=None):
        T, X, k = step.rows, self.experts, self.top_k
        z = step.buf("experts.router_logits", (T, X), torch.float32)
        slices = ops.gemm_f32_slices(X, h32.shape[1])
        parts = step.buf("experts.router_parts", (slices, T, X), torch.float32) if slices > 1 else None
        ops.gemm_f32(h32, self.w_router, z, parts=parts)
        ids = step.buf("experts.ids", (T, k), torch.int32)
        weights = step.buf("experts.weights", (T, k), torch.float32)
        counts = step.buf("experts.counts", (X,), torch.int32)
        offsets = step.buf("experts.offsets", (X + 1,), torch.int32)
        pairs = step.buf("experts.pairs", (T * k,), torch.int32)
        active = step.buf("experts.active", (X,), torch.int32)
        n_active = step.buf("experts.n_active", (1,), torch.int32)
        need = ops.moe_align_scratch(T * k, X)
        scratch = step.buf("experts.align_scratch", (need,), torch.int32) if need else None
        # for steps of many pairs the grouping also counts the experts' tiles of 128 rows, by which the products choose their tiles
        tile_stats = step.buf("experts.tile_stats", (1,), torch.int32) if T * k >= ops.TILE_STATS_MIN_PAIRS else None
        ops.route_topk_align(z, self.bias, ids, weights, k, self.score, self.normalize, self.scale, counts, offsets, pairs, active, n_active,
                             parts=parts, scratch=scratch, tile_stats=tile_stats)
        step.observe("routing", logits=z, ids=ids, weights=weights)
        act = step.buf("experts.act", (T * k, self.intermediate), step.act_dtype)
        ops.grouped_gemm(h, self.w_gate_up, act, offsets, pairs, k, ops.EPI_SWIGLU, active, n_active, token_rows=T, tile_stats=tile_stats)
        y = step.buf("experts.y", (T * k, self.hidden), torch.float32)
        ops.grouped_gemm(act, self.w_down, y, offsets, pairs, 1, ops.EPI_STORE, active, n_active, token_rows=T, tile_stats=tile_stats)
        ops.moe_combine(out, y, ids, weights, accumulate)


class DenseGLU(FeedForward):
    """params: hidden, intermediate.  y = (silu(h.Wg^T) * (h.Wu^T)).Wd^T; tensors gate_proj, up_proj, down_proj (.weight)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        self.w_gate_up = self.w_down = None

    def tensor_specs(self, available):
        F, E = self.intermediate, self.hidden
        fused = self.name("gate_up_proj.weight")     # gate rows, then up rows, filled from the file's two tensors
        return [TensorSpec(self.name("gate_proj.weight"), (F, E), into=(fused, (2 * F, E), (slice(0, F),))),
                TensorSpec(self.name("up_proj.weight"), (F, E), into=(fused, (2 * F, E), (slice(F, 2 * F),))),
                TensorSpec(self.name("down_proj.weight"), (E, F))]

    def load(self, tensors):
        self.w_gate_up = tensors[self.name("gate_up_proj.weight")]
        self.w_down = tensors[self.name("down_proj.weight")]

    def takes_deferred_norm(self, step):
        return ops.gemm_takes_normed_rows(step.rows, self.w_gate_up, step.act_dtype, ops.EPI_SWIGLU)

    def forward(self, step, h, out, accumulate, h32=None):
        act = step.buf("glu.act", (step.rows, self.intermediate), step.act_dtype)
        ops.gemm(h, self.w_gate_up, act, ops.EPI_SWIGLU)
        ops.gemm(act, self.w_down, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("feed_forward", "routed_experts", RoutedExperts)
register("feed_forward", "dense_glu", DenseGLU)
