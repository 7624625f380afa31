"""Causal grouped-query softmax attention over the paged cache.

Per row: q, k, v projections of the normed input (no biases); an optional RMSNorm over the whole q and the whole k
projection; rotation of the first `rotary_dim` values of each head at the row's position; k and v written to the
request's pages; softmax(q.k * head_dim^-1/2) over keys 0..p (or the last `window`) of the same request, head h reading
KV head h / (heads / kv_heads); output projection.  Formula order: /root/reference/src/backends/cpu/cpu_backend.hpp:971-1104
(attention), :1461-1480 (rotation); the norm over the whole projection is this architecture's variant of the
reference's per-head norm (/root/reference/src/model/arch/minimax_m3.hpp:258-259).
"""

from __future__ import annotations

import numpy as np
import torch

from .. import ops
from ..limits import MAX_HEAD_DIM
from .base import BuildContext, LayerCache, Mixer, build_part, register
from .spec import KVNeed, PartSpec, TensorSpec

_NORM_MODES = {"none": ops.QKNORM_NONE, "projection": ops.QKNORM_PROJECTION}


class Attention(Mixer):
    """params: hidden, heads, kv_heads, head_dim, qk_norm ("projection" | "none"), eps, window (None | int), position (PartSpec),
    scale (None: head_dim^-1/2; else the factor the scores are multiplied by)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden = int(p["hidden"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.eps = float(p.get("eps", 0.0))
        self.window = p.get("window")
        if self.heads % self.kv_heads:
            raise ValueError("the head count must be divisible by the KV head count")
        if not 0 < self.head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"attention: head_dim {self.head_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        if p.get("qk_norm", "none") not in _NORM_MODES:
            raise ValueError(f"qk_norm {p.get('qk_norm')!r} is not one of {sorted(_NORM_MODES)}")
        self.norm_mode = _NORM_MODES[p.get("qk_norm", "none")]
        self.position = build_part("position", p.get("position") or PartSpec("none"), ctx)
        pairing = getattr(self.position, "pairing", "halves")
        if pairing not in ("halves", "interleaved"):
            raise ValueError(f"attention: rotary pairing {pairing!r} is not one the kernels rotate (halves, interleaved)")
        self.pairing = ops.ROPE_INTERLEAVED if pairing == "interleaved" else ops.ROPE_HALVES
        # softmax(q.k * scale): head_dim^-1/2 unless the architecture gives its own
        self.scale = float(p["scale"]) if p.get("scale") is not None else float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim)))
        if not self.scale > 0.0:
            raise ValueError(f"attention: the softmax scale must be positive, not {self.scale}")
        self.q_width = self.heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.wqkv = self.wo = self.q_norm = self.k_norm = None

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def tensor_specs(self, available):
        # one product for the three projections: the file's q, k and v go straight into the rows q | k | v of one tensor
        fused, shape = self.name("qkv_proj.weight"), (self.q_width + 2 * self.kv_width, self.hidden)
        q, kv = self.q_width, self.kv_width
        specs = [
            TensorSpec(self.name("q_proj.weight"), (q, self.hidden), into=(fused, shape, (slice(0, q),))),
            TensorSpec(self.name("k_proj.weight"), (kv, self.hidden), into=(fused, shape, (slice(q, q + kv),))),
            TensorSpec(self.name("v_proj.weight"), (kv, self.hidden), into=(fused, shape, (slice(q + kv, q + 2 * kv),))),
            TensorSpec(self.name("o_proj.weight"), (self.hidden, self.q_width)),
        ]
        if self.norm_mode == ops.QKNORM_PROJECTION:
            specs += [TensorSpec(self.name("q_norm.weight"), (self.q_width,), "norm"),
                      TensorSpec(self.name("k_norm.weight"), (self.kv_width,), "norm")]
        return specs

    def load(self, tensors):
        self.wqkv = tensors[self.name("qkv_proj.weight")]
        self.wo = tensors[self.name("o_proj.weight")]
        if self.norm_mode == ops.QKNORM_PROJECTION:
            self.q_norm = tensors[self.name("q_norm.weight")]
            self.k_norm = tensors[self.name("k_norm.weight")]

    def takes_deferred_norm(self, step):
        return ops.gemm_takes_normed_rows(step.rows, self.wqkv, torch.float32)

    def _plan(self, step):
        """The matrix-core attention kernel's work items for this step's rows: made once a step and shared by every
        layer with the same heads and window."""
        window = int(self.window or 0)
        return step.shared(("attention.plan", self.heads, self.kv_heads, window),
                           lambda: ops.attention_plan([e.n for e in step.entries], [e.past + e.n for e in step.entries], self.heads,
                                                      self.kv_heads, step.device, window))

    def graph_key(self, step):
        # a recorded step holds the plan's addresses and launch sizes; the universal kernel has no plan
        page = self.ctx.page_tokens
        return self._plan(step) if page and ops.attention_mfma_ok(step.act_dtype, self.head_dim, page) else None

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T = step.rows
        act = step.act_dtype
        qkv = step.buf("attention.qkv", (T, self.q_width + 2 * self.kv_width), torch.float32)
        ops.gemm(h, self.wqkv, qkv, scratch=step.buf)
        q = step.buf("attention.q", (T, self.q_width), act)
        cos_sin, rotary = self.position.rotation()
        tables = step.tables(cache.group)
        ops.qknorm_rope_kvwrite(qkv, self.q_norm, self.k_norm, cos_sin, step.positions, step.row_entry, tables, q, cache.k, cache.v,
                                self.eps, self.heads, self.kv_heads, self.head_dim, rotary, self.norm_mode, write_kv=cache.writes,
                                pairing=self.pairing)
        o = step.buf("attention.out", (T, self.q_width), act)
        plan = self._plan(step) if ops.attention_mfma_ok(act, self.head_dim, cache.k.shape[2]) else None
        ops.paged_attention(q, cache.k, cache.v, step.positions, step.row_entry, tables, o, self.scale, self.heads,
                            window=int(self.window or 0), plan=plan, scratch=step.buf)
        ops.gemm(o, self.wo, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "attention", Attention)
