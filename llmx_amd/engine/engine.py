"""The engine: a built model, its cache on the device, and the one step function everything else drives.

`step` takes a batch of (request, its next tokens): portions of prompts beside single decoded tokens, cut anywhere.
It runs only the tokens it is given, as one batch, from the cache earlier steps left, and returns the logits at the
wanted places.  The transaction follows the reference's pass (/root/reference/src/model/passes.hpp:271-413 refusals
before anything is reserved, :633-653 reserve pages, :771-830 run, :1007-1032 commit, :1124-1134 roll back).
"""

from __future__ import annotations

from dataclasses import replace
from pathlib import Path
from typing import Dict, Hashable, List, Optional, Sequence, Union

import numpy as np
import torch

from .. import ops
from ..cache import CacheManager, GroupSpec, OutOfPages
from ..models import registry
from ..parts.base import BuildContext, LayerCache, Part
from ..parts.spec import ModelSpec, PagedNeed, StateNeed
from ..weights import ModelFiles, RandomInit, load as load_weights
from ..weights.loader import device_dtype
from ..weights.random_init import fill_random, stored_dtype
from .batch import EntryView, RowPlanUploader, StepEntry, StepError, StepState, Workspace, check_entries
from .model import BuiltModel

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def resolve_dtype(dtype: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype in (torch.float32, torch.bfloat16):
            return dtype
    elif dtype in _DTYPES:
        return _DTYPES[dtype]
    raise ValueError(f"dtype {dtype!r} is not float32 or bfloat16")


class _StepGraph:
    """A recorded decode step: the graph, where its logits appear, and what must not have moved since."""

    def __init__(self, graph, logits, shared, workspace_generation, uploader_generation):
        self.graph = graph
        self.logits = logits
        self.shared = shared    # kept alive: what the parts made for the step (work plans the graph's kernels read)
        self.generations = (workspace_generation, uploader_generation)

    def stale(self, engine: "Engine") -> bool:
        return self.generations != (engine._workspace.generation, engine._uploader.generation)


class Engine:
    def __init__(self, config, spec: ModelSpec, dtype: Union[str, torch.dtype] = "bfloat16", *, kv_tokens: int,
                 page_tokens: int = 16, max_requests: int = 8, device: Union[str, torch.device] = "cuda:0", weights=None,
                 graphs: bool = True, step_tokens: Optional[int] = None):
        """`weights(engine)` returns the device tensors by name; it runs before the cache is allocated, so weights that
        do not fit the model are refused before anything large exists.  `graphs`: steps of single decoded tokens are
        replayed as HIP graphs once their shape has been seen twice (see `_run`).  `step_tokens`: the most tokens a
        step brings of one request, when the caller keeps to one (a scheduler's budget): a cache group that keeps only
        a window of keys then gets a pool for `max_requests` windows instead of `kv_tokens` tokens; a step that brings
        more finds the pool short and is refused like any step that runs out of pages."""
        if not torch.cuda.is_available():
            raise RuntimeError("llmx_amd runs on a GPU only: no GPU is visible and there is no CPU path")
        ops.lib()  # fail now, loudly, when the kernel library is missing
        self.config = config
        self.spec = spec
        self.device = torch.device(device)
        self.act_dtype = resolve_dtype(dtype)
        if page_tokens <= 0 or kv_tokens <= 0:
            raise ValueError("page_tokens and kv_tokens must be positive")
        self.page_tokens = int(page_tokens)
        self.kv_tokens = -(-int(kv_tokens) // self.page_tokens) * self.page_tokens
        self.max_requests = int(max_requests)
        if step_tokens is not None and step_tokens < 1:
            raise ValueError("step_tokens must be at least 1")
        self.step_tokens = step_tokens
        self.max_positions = min(spec.max_positions, self.kv_tokens)
        torch.cuda.set_device(self.device)
        ctx = BuildContext(self.act_dtype, self.device, self.max_positions, self.page_tokens)
        self.model = BuiltModel(spec, ctx)
        self._loaded = False
        if weights is not None:
            self.model.load(weights(self))
            self._loaded = True
        self._workspace = Workspace(self.device)
        self._uploader = RowPlanUploader(self.device)
        #: callable(step, kind, **tensors): sees what parts show of a step (the reference's route hook,
        #: /root/reference/src/model/arch/blocks.hpp:118-138); None in serving
        self.observer = None
        self._make_cache()
        self.graphs = bool(graphs) and all(getattr(p, "graph_safe", False) for p in self.model.parts()) \
            and all(getattr(b, "graph_safe", False) for b in self.model.blocks)
        self._graphs: Dict[tuple, "_StepGraph"] = {}
        self._graph_seen: Dict[tuple, int] = {}
        # the parts that have a say in a recorded step's key (see Part.graph_key)
        self._keyed_parts = [p for p in self.model.parts() if type(p).graph_key is not Part.graph_key]
        self.graph_replays = 0                # steps that ran as a replay (for tests and measurement)

    # -- construction -----------------------------------------------------------
    @classmethod
    def load(cls, folder: Union[str, Path], dtype="bfloat16", **options) -> "Engine":
        """An engine for the model folder (config.json + safetensors); the model class is chosen by config.json."""
        config, spec = registry.read_model_dir(folder)
        files = ModelFiles(folder)

        def from_files(eng: "Engine"):
            specs = eng.model.tensor_specs(set(files.names()))
            return load_weights(specs, files, eng.device, eng.act_dtype == torch.float32)

        try:
            return cls(config, spec, dtype, weights=from_files, **options)
        finally:
            files.close()

    @classmethod
    def from_random(cls, config, init: RandomInit = RandomInit(), dtype="bfloat16", tensors_out: Optional[dict] = None,
                    **options) -> "Engine":
        """An engine whose weights are generated on the device from (seed, tensor name); nothing is read or written.
        `tensors_out`, when given, receives the device tensors by the names a model folder would hold (a tensor that
        is a slice of a fused one as a view of it) and the fused tensors by the names the parts read them under."""
        def generate(eng: "Engine"):
            tensors, by_file_name = {}, {}
            for s in eng.model.tensor_specs():
                dt = device_dtype(s, stored_dtype(s, init), eng.act_dtype == torch.float32)
                if s.into is None:
                    t = tensors[s.name] = torch.empty(s.shape, dtype=dt, device=eng.device)
                else:   # a slice of a fused tensor, filled in place with the values its own name gives
                    target, shape, index = s.into
                    if target not in tensors:
                        tensors[target] = torch.empty(shape, dtype=dt, device=eng.device)
                    t = tensors[target][index]
                    if not t.is_contiguous() or tuple(t.shape) != tuple(s.shape):
                        raise ValueError(f"random weights: {s.name} is not a contiguous slice of {target}")
                fill_random(t, s, init)
                by_file_name[s.name] = t
            if tensors_out is not None:
                tensors_out.update(tensors)
                tensors_out.update(by_file_name)
            return tensors

        return cls(config, registry.assemble(config), dtype, weights=generate, **options)

    def _make_cache(self) -> None:
        """Allocates what the mixers' needs list: for every group of equal paged needs a page pool and, for each of the
        need's tensors, one arena [caches of the group, pages, *page shape]; for every state need [slots, *shape]."""
        needs = self.model.cache_needs()
        n_pages = self.kv_tokens // self.page_tokens
        keys: List[PagedNeed] = []
        self._group_of: List[int] = []          # cache number -> group (or -1)
        self._index_in_group: List[int] = []
        counts: List[int] = []
        for need in needs:
            if isinstance(need, PagedNeed):
                if need not in keys:
                    keys.append(need)
                    counts.append(0)
                g = keys.index(need)
                self._group_of.append(g)
                self._index_in_group.append(counts[g])
                counts[g] += 1
            else:
                self._group_of.append(-1)
                self._index_in_group.append(-1)
        self.group_needs = keys
        groups = [GroupSpec(f"kv{g}", self.page_tokens, n_pages, need.window) for g, need in enumerate(keys)]
        groups = [replace(g, n_pages=g.pool_pages(self.kv_tokens, self.max_requests, self.step_tokens)) for g in groups]
        # a model with per-request state steps into a second slot, so that a step that fails leaves the state as it was
        self._stateful = any(isinstance(need, StateNeed) for need in needs)
        self.cache = CacheManager(groups, self.max_requests, shadow_slots=self._stateful)
        self._paged: List[Dict[str, torch.Tensor]] = []
        for g, need in enumerate(keys):
            self._paged.append({t.name: torch.zeros((counts[g], groups[g].n_pages, *t.page_shape(self.page_tokens)),
                                                    dtype=getattr(torch, t.dtype) if t.dtype else self.act_dtype, device=self.device)
                                for t in need.tensors})
        self._state: List[Optional[torch.Tensor]] = []
        for need in needs:
            if isinstance(need, StateNeed):
                self._state.append(torch.zeros((self.cache.slots.capacity, *need.shape), dtype=getattr(torch, need.dtype), device=self.device))
            else:
                self._state.append(None)
        self._layer_caches: List[LayerCache] = []
        for e in self.spec.run_order:
            g = self._group_of[e.cache]
            if g >= 0:
                at = self._index_in_group[e.cache]
                self._layer_caches.append(LayerCache(group=g, tensors={name: arena[at] for name, arena in self._paged[g].items()},
                                                     writes=e.writes))
            else:
                self._layer_caches.append(LayerCache(state=self._state[e.cache], writes=e.writes))

    # -- requests ---------------------------------------------------------------
    def add_request(self, request: Hashable) -> int:
        """Opens a request: a state slot is taken and its state cleared; pages come with its first tokens."""
        slot = self.cache.open(request)
        for s in self._state:
            if s is not None:
                s[slot].zero_()
        return slot

    def end_request(self, request: Hashable) -> None:
        """The request is finished: what it holds is given back."""
        self.cache.close(request)

    def truncate(self, request: Hashable, length: int) -> None:
        """Takes the request back to its first `length` tokens (its pages beyond them are given back), so that it can go
        on from that prefix: scoring another continuation, dropping a rejected draft.  A model that keeps fixed-size
        state per request can only be taken back to nothing (the state is cleared) or left as it is: a state cannot be
        unwound.  The reference's rule: /root/reference/src/model/kv_cache.hpp:126-134, history.hpp:58-59."""
        held = self.cache.length(request)
        if self._stateful and 0 < length < held:
            raise StepError(f"truncate: request {request!r} keeps a state of fixed size, which cannot be taken back to {length} of {held} tokens")
        self.cache.truncate(request, length)
        if self._stateful and length == 0 and held > 0:
            slot = self.cache.slot(request)
            for s in self._state:
                if s is not None:
                    s[slot].zero_()

    def has_request(self, request: Hashable) -> bool:
        return self.cache.is_open(request)

    def length(self, request: Hashable) -> int:
        return self.cache.length(request)

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    # -- the step ---------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits [wanted, vocab] in the order of entries and `want`.

        The returned tensor is scratch storage: it is valid until the next step.
        """
        if not self._loaded:
            raise RuntimeError("the engine has no weights yet")
        entries = list(entries)
        views = check_entries(entries, self.cache, self.max_positions, self.spec.vocab_size)
        T = views[-1].row0 + views[-1].n

        prepared: List[Hashable] = []
        try:
            for e, v in zip(entries, views):
                self.cache.prepare(e.request, v.n)
                prepared.append(e.request)
        except OutOfPages:
            for r in prepared:
                self.cache.abort(r)
            raise
        try:
            if self._stateful:
                views = self._enter_shadow_slots(views)
            logits = self._run(entries, views, T)
        except BaseException:
            for r in prepared:
                self.cache.abort(r)
            raise
        for r in prepared:
            self.cache.commit(r)
        return logits

    def _enter_shadow_slots(self, views: List[EntryView]) -> List[EntryView]:
        """Each entry's state is copied into the slot its step writes, and the entry is pointed there; the slot it had
        is not touched until the step commits."""
        moved = []
        for v in views:
            to = self.cache.step_slot(v.request)
            if to != v.slot:
                for s in self._state:
                    if s is not None:
                        s[to].copy_(s[v.slot])
            moved.append(replace(v, slot=to))
        return moved

    # -- wrappers over step, for one request (the reference's Model::prefill / step / score, runtime.hpp:1278-1385) --
    def prefill(self, request: Hashable, tokens: Sequence[int], portion: int = 512) -> torch.Tensor:
        """Feeds `tokens` in portions of at most `portion`; returns the float32 logits [vocab] after the last token."""
        tokens = list(tokens)
        if not tokens:
            raise StepError("prefill: no tokens")
        if portion < 1:
            raise StepError("prefill: a portion holds at least one token")
        row = None
        for s in range(0, len(tokens), portion):
            part = tokens[s:s + portion]
            last = s + len(part) == len(tokens)
            out = self.step([StepEntry(request, part, [len(part) - 1] if last else [])])
            if last:
                row = out[0]
        return row

    def decode_one(self, request: Hashable, token: int) -> torch.Tensor:
        """Feeds one token; returns the float32 logits [vocab] after it."""
        return self.step([StepEntry(request, [int(token)], [0])])[0]

    def score(self, request: Hashable, tokens: Sequence[int], portion: int = 512, each=None) -> Optional[torch.Tensor]:
        """The logits at every position of `tokens`, fed in portions.

        With `each`, it is called as each(first_position, logits [n, vocab]) per portion (the storage is reused by
        the next one) and nothing is returned; without, the rows come back as one float32 tensor [len(tokens), vocab].
        """
        tokens = list(tokens)
        if not tokens:
            raise StepError("score: no tokens")
        if portion < 1:
            raise StepError("score: a portion holds at least one token")
        rows = None if each else torch.empty(len(tokens), self.spec.vocab_size, dtype=torch.float32, device=self.device)
        for s in range(0, len(tokens), portion):
            part = tokens[s:s + portion]
            out = self.step([StepEntry(request, part, list(range(len(part))))])
            if each:
                each(s, out)
            else:
                rows[s:s + len(part)] = out
        return rows

    def _run(self, entries: List[StepEntry], views: List[EntryView], T: int) -> torch.Tensor:
        n_e = len(entries)
        token_ids = np.empty(T, dtype=np.int32)
        positions = np.empty(T, dtype=np.int32)
        row_entry = np.empty(T, dtype=np.int32)
        pick: List[int] = []
        for i, (e, v) in enumerate(zip(entries, views)):
            token_ids[v.row0:v.row0 + v.n] = np.asarray(e.tokens, dtype=np.int32)
            positions[v.row0:v.row0 + v.n] = np.arange(v.past, v.past + v.n, dtype=np.int32)
            row_entry[v.row0:v.row0 + v.n] = i
            pick.extend(v.row0 + int(w) for w in e.want)
        slots = np.asarray([v.slot for v in views], dtype=np.int32)
        arrays = [token_ids, positions, row_entry, slots, np.asarray(pick if pick else [0], dtype=np.int32)]
        for g in range(len(self.cache.groups)):
            tables = [self.cache.table(e.request, g) for e in entries]
            width = max(1, max(len(t) for t in tables))
            width = -(-width // 64) * 64     # in steps of 64 pages, so that a growing context keeps its width (and its graph) for long
            packed = np.full((n_e, width), -1, dtype=np.int32)
            for i, t in enumerate(tables):
                packed[i, :len(t)] = t
            arrays.append(packed)
        dev = self._uploader.upload(arrays)

        step = StepState(self._workspace, self.act_dtype)
        step.rows = T
        step.entries = views
        step.token_ids, step.positions, step.row_entry, step.entry_slots = dev[0], dev[1], dev[2], dev[3]
        step.pick = dev[4][:len(pick)]
        step._tables = dev[5:]
        step.max_rows_per_entry = max(v.n for v in views)
        step.observer = self.observer

        # A step of single decoded tokens launches a few hundred short kernels; replayed as one HIP graph they follow
        # each other without the host.  A graph holds addresses and launch sizes, so it is keyed by all that fixes
        # them (rows, wanted places, widths of the block tables, what the parts add: Part.graph_key) and dropped when
        # scratch storage moves.  The row plan is copied to the device before the replay, outside the graph; the graph holds kernels only.
        key = None
        if self.graphs and self.observer is None and len(pick) > 0 and all(v.n == 1 for v in views):
            key = (T, tuple(pick), tuple(a.shape for a in arrays[5:]), tuple(p.graph_key(step) for p in self._keyed_parts))
            graph = self._graphs.get(key)
            if graph is not None and not graph.stale(self):
                graph.graph.replay()
                self.graph_replays += 1
                self._uploader.mark()
                return graph.logits
            if graph is not None:
                self._graphs.clear()
                self._graph_seen.clear()
        if key is not None and self._graph_seen.get(key, 0) >= 1:
            graph = self._capture(step, key)
            if graph is not None:
                graph.graph.replay()
                self.graph_replays += 1
                self._uploader.mark()
                return graph.logits
        logits = self._forward(step)
        if key is not None:
            if len(self._graph_seen) > 256:
                self._graph_seen.clear()
            self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
        return logits

    def _forward(self, step: StepState) -> torch.Tensor:
        T, E = step.rows, self.spec.hidden_size
        x = step.buf("residual", (T, E), torch.float32)
        self.model.embedding.forward(step, x)
        for i, (entry, cache) in enumerate(zip(self.spec.run_order, self._layer_caches)):
            step.run_index = i
            self.model.blocks[entry.layer].forward(step, x, cache)
        W = step.pick.shape[0]
        if W == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        rows = step.buf("head.rows", (W, E), self.act_dtype)
        self.model.final_norm.forward(step, x, rows, None, step.pick)
        logits = step.buf("logits", (W, self.spec.vocab_size), torch.float32)
        self.model.head.forward(step, rows, logits)
        return logits

    def _capture(self, step: StepState, key: tuple) -> Optional["_StepGraph"]:
        """Records the step's launches (a step of this shape ran before, so every scratch tensor exists) into a graph."""
        before = (self._workspace.generation, self._uploader.generation)
        graph = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(graph):
                logits = self._forward(step)
        except Exception as err:   # a graph is an optimisation: without it the step runs as it always did
            import warnings
            warnings.warn(f"llmx_amd: recording a decode step as a HIP graph failed ({err}); steps run without graphs")
            self.graphs = False
            return None
        if (self._workspace.generation, self._uploader.generation) != before:
            return None            # storage moved while recording: the graph holds stale addresses
        if len(self._graphs) >= 32:
            self._graphs.pop(next(iter(self._graphs)))
        record = _StepGraph(graph, logits, dict(step._shared), *before)
        self._graphs[key] = record
        return record

    # -- accounting -------------------------------------------------------------
    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for p in self.model.parts():
            for v in vars(p).values():
                if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                    seen.add(v.data_ptr())
                    total += v.numel() * v.element_size()
        return total

    def cache_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for arenas in self._paged for t in arenas.values()) + sum(t.numel() * t.element_size() for t in self._state if t is not None)
