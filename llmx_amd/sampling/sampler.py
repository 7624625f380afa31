"""Draws the next token of each wanted row on the device.

Order of operations as the reference's sampler (/root/reference/src/inference/sampler.hpp:258-378): penalties from the
raw logit, then greedy, or top-k, top-p, min-p and the draw; one uniform number is taken from the request's generator
per sampled (non-greedy) row, before the branch.
"""

from __future__ import annotations

from collections import Counter
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import MAX_EXACT_TOP_K, SamplingParams, XorShift64


class _Seen:
    """The distinct tokens of one request's history and how often each was seen, kept up as the history grows."""

    __slots__ = ("n", "index", "ids", "counts")

    def __init__(self):
        self.n, self.index, self.ids, self.counts = 0, {}, [], []

    def follow(self, history: Sequence[int]) -> None:
        if len(history) < self.n:      # the history was cut: count again
            self.__init__()
        for tok in history[self.n:]:
            at = self.index.get(tok)
            if at is None:
                self.index[tok] = len(self.ids)
                self.ids.append(tok)
                self.counts.append(1)
            else:
                self.counts[at] += 1
        self.n = len(history)


class Sampler:
    def __init__(self, vocab_size: int, device: torch.device):
        self.vocab = vocab_size
        self.device = device
        self._kept = None     # (key, settings) of the last rows sampled
        self._seen = {}       # request key -> _Seen, for the rows whose penalties need their histories' counts
        self._unit_host = self._unit_dev = None    # the rows' uniform numbers: pinned host memory and its place on the device

    def _f32(self, values) -> torch.Tensor:
        return torch.tensor(np.asarray(values, dtype=np.float32), device=self.device)

    def _units(self, values) -> torch.Tensor:
        """The step's uniform numbers on the device, copied from pinned memory without waiting for the stream: the copy and
        the sampling kernels queue up behind the step while it still runs.  (A copy from pageable memory would hold the
        host until the step is over, and the kernels' launches would then follow it with the device idle.)  The buffers
        are free again when a call's tokens have been read back, which every call that uses them ends with."""
        W = len(values)
        if self._unit_host is None or self._unit_host.numel() < W:
            n = max(64, 2 * W)
            self._unit_host = torch.empty(n, dtype=torch.float32, pin_memory=True)
            self._unit_dev = torch.empty(n, dtype=torch.float32, device=self.device)
        self._unit_host[:W] = torch.from_numpy(np.asarray(values, dtype=np.float32))
        self._unit_dev[:W].copy_(self._unit_host[:W], non_blocking=True)
        return self._unit_dev[:W]

    def _i32(self, values) -> torch.Tensor:
        return torch.tensor(np.asarray(values, dtype=np.int32), device=self.device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], generated: Sequence[Sequence[int]],
               rngs: Sequence[XorShift64], eos: Optional[int], keys: Optional[Sequence] = None) -> List[int]:
        """One token id for each row of `logits` [W, vocab]; `generated` holds each row's tokens so far (for the penalties).

        The logits are scratch of the step and are changed in place by the penalties.  `keys` (one hashable a row, a
        request's id for instance): a row's history is the history the same key had at the last call, grown at its end;
        its counts are then kept up token by token instead of being formed again from the whole history at every step.
        """
        W = logits.shape[0]
        if not (len(params) == len(generated) == len(rngs) == W) or (keys is not None and len(keys) != W):
            raise ValueError("sampler: one set of settings, one history and one generator per row")
        if W == 0:
            return []
        # penalties, in place: one list entry per (row, distinct seen token)
        rows, ids, counts = [], [], []
        seen_now = {}
        for r, (p, gen) in enumerate(zip(params, generated)):
            if p.penalized and gen:
                if keys is None:
                    seen = Counter(gen)
                    row_ids, row_counts = list(seen.keys()), list(seen.values())
                else:
                    seen = seen_now[keys[r]] = self._seen.get(keys[r]) or _Seen()
                    seen.follow(gen)
                    row_ids, row_counts = seen.ids, seen.counts
                rows += [r] * len(row_ids)
                ids += row_ids
                counts += row_counts
        self._seen = seen_now     # requests that are no longer sampled are forgotten
        if rows:
            ops.penalize(logits, self._i32(rows), self._i32(ids), self._i32(counts), self._f32([p.penalty for p in params]),
                         self._f32([p.presence_penalty for p in params]), self._f32([p.frequency_penalty for p in params]))
        st = self._settings(params, eos)
        skip = st["skip"]
        out = torch.empty(W, dtype=torch.int32, device=self.device)
        if st["greedy"]:
            ops.argmax_rows(logits, out, skip)
            return out.tolist()
        unit = self._units([0.0 if p.greedy else rng.unit() for p, rng in zip(params, rngs)])
        temp, min_p, which = st["temp"], st["min_p"], st["which"]
        results = {}
        if "all" in which:
            ops.sample_all(logits, temp, unit, out, min_p, skip)
            results["all"] = out
        if "topk" in which:
            results["topk"] = torch.zeros(W, dtype=torch.int32, device=self.device)
            ops.sample_topk(logits, temp, st["top_k"], st["top_p"], min_p, unit, results["topk"], skip, max_keep=st["max_keep"])
        if "ranked" in which:
            results["ranked"] = torch.zeros(W, dtype=torch.int32, device=self.device)
            ops.sample_ranked(logits, temp, st["top_k"], st["top_p"], min_p, unit, results["ranked"], skip, slices=st["nucleus_rows"])
        if len(results) == 1:
            return next(iter(results.values())).tolist()
        lists = {name: t.tolist() for name, t in results.items()}
        return [lists[name][row] for row, name in enumerate(which)]

    def _settings(self, params: Sequence[SamplingParams], eos: Optional[int]) -> dict:
        """The rows' settings as device tensors, and which kernel takes each row.  They change only when the set of
        running requests does, so the last set is kept: a decode loop then uploads one tensor a step (the uniforms)."""
        key = (eos, tuple((p.temp, p.top_k, p.top_p, p.min_p, p.ignore_eos) for p in params))
        if self._kept is not None and self._kept[0] == key:
            return self._kept[1]
        st = {"greedy": all(p.greedy for p in params), "skip": None}
        if eos is not None and any(p.ignore_eos for p in params):
            st["skip"] = self._i32([eos if p.ignore_eos else -1 for p in params])
        if not st["greedy"]:
            # ids a draw can give: all, less a masked end token; a top_k that leaves them all is no top_k
            m = [self.vocab - (1 if (eos is not None and p.ignore_eos and 0 <= eos < self.vocab and self.vocab > 1) else 0) for p in params]

            # which kernel takes a row: everything kept and no nucleus: the walk over the whole row; a top-k of at most
            # MAX_EXACT_TOP_K: ranked whole in LDS; anything else (a larger top-k, a nucleus over the whole row): the
            # search by histograms.  With mixed settings each kernel in use runs over all rows and a row takes the
            # result of its own.
            def kernel_of(p, mr):
                if p.greedy or ((p.top_k <= 0 or p.top_k >= mr) and p.top_p >= 1.0):
                    return "all"
                return "topk" if 0 < p.top_k <= MAX_EXACT_TOP_K else "ranked"
            st["which"] = [kernel_of(p, mr) for p, mr in zip(params, m)]
            st["temp"] = self._f32([p.temp for p in params])
            st["min_p"] = self._f32([p.min_p for p in params])
            if "topk" in st["which"] or "ranked" in st["which"]:
                st["top_k"], st["top_p"] = self._i32([p.top_k for p in params]), self._f32([p.top_p for p in params])
                # the largest top_k among the rows the exact kernel takes: it sizes that kernel's candidate lists
                st["max_keep"] = max([p.top_k for p, w in zip(params, st["which"]) if w == "topk"] or [1])
                # a nucleus over a whole row is first looked for by slices; a top-k above what is ranked whole never is
                st["nucleus_rows"] = any(w == "ranked" and (p.top_k <= 0 or p.top_k >= mr) for p, w, mr in zip(params, st["which"], m))
        self._kept = (key, st)
        return st
