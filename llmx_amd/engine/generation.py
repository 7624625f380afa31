"""Generation: the scheduler driving the engine's step function and the device sampler.

The loop is the reference's generate (/root/reference/src/inference/generate.hpp:19-124) for many requests at once:
the first token comes from the logits of the prompt's last row, every later one from a one-token step; an end token is
neither kept nor fed; at max_tokens the request ends.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence

from ..sampling.params import SamplingParams, XorShift64
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .engine import Engine
from .scheduler import DEFAULT_STEP_TOKENS, PlannedEntry, Request, Scheduler, SchedulerError


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    steps: int = 0
    prompt_seconds: float = 0.0     # time of steps that carried prompt portions
    decode_seconds: float = 0.0     # time of steps that carried only decoded tokens
    decode_steps: int = 0           # such steps
    decode_rows: int = 0            # and the tokens they carried


class Generator:
    """Owns a scheduler and a sampler over one engine; `run` plays every submitted request to its end."""

    def __init__(self, engine: Engine, max_seqs: Optional[int] = None, max_step_tokens: int = DEFAULT_STEP_TOKENS,
                 feed_last: bool = True):
        self.engine = engine
        self.scheduler = Scheduler(engine.cache.groups, max_seqs or engine.max_requests, max_step_tokens,
                                   max_positions=engine.max_positions, eos_token_id=engine.spec.eos_token_id, feed_last=feed_last)
        if self.scheduler.max_seqs > engine.max_requests:
            raise SchedulerError(f"generation: {self.scheduler.max_seqs} seats but the engine holds {engine.max_requests} requests")
        self.sampler = Sampler(engine.vocab_size, engine.device)
        self.stats = GenerationStats()

    def submit(self, request: Request) -> None:
        V = self.engine.vocab_size
        for t in request.prompt:
            if not 0 <= int(t) < V:
                raise SchedulerError(f"generation: token id {t} is outside the vocabulary")
        self.scheduler.submit(request)

    def step(self, on_token: Optional[Callable[[Hashable, int], None]] = None) -> List[Request]:
        """One round: admit, plan, run, sample, advance.  Returns the requests that finished in it.

        When the round fails (a refused step, a kernel error) every running request is ended in the engine before the
        error goes on, and retired in the scheduler (finish reason "error", its reservation returned), so that nothing stays open holding a
        slot and pages and the generator can go on with the requests that wait."""
        try:
            return self._round(on_token)
        except BaseException:
            for r in self.scheduler.fail_running():
                if self.engine.has_request(r.id):
                    self.engine.end_request(r.id)
            raise

    def _round(self, on_token: Optional[Callable[[Hashable, int], None]]) -> List[Request]:
        sch = self.scheduler
        for r in sch.admit():
            self.engine.add_request(r.id)
        plan = sch.plan()
        if not plan:
            if sch.running or sch.waiting:
                raise SchedulerError("generation: nothing to run while requests are waiting; the cache cannot hold the next one")
            return []
        t0 = time.perf_counter()
        entries = [StepEntry(e.request, e.tokens, [len(e.tokens) - 1] if e.wants_logits else []) for e in plan]
        logits = self.engine.step(entries)
        wanting = [e for e in plan if e.wants_logits]
        by_id = {r.id: r for r in sch.running}
        reqs = [by_id[e.request] for e in wanting]
        tokens = self.sampler.sample(logits, [r.params for r in reqs], [r.generated for r in reqs], [r.rng for r in reqs],
                                     self.engine.spec.eos_token_id, keys=[r.id for r in reqs])
        dt = time.perf_counter() - t0
        prompt_rows = sum(len(e.tokens) for e in plan if len(e.tokens) > 1 or not by_id[e.request].generated)
        self.stats.steps += 1
        if prompt_rows:
            self.stats.prompt_seconds += dt
            self.stats.prompt_tokens += prompt_rows
        else:
            self.stats.decode_seconds += dt
            self.stats.decode_steps += 1
            self.stats.decode_rows += len(plan)
        sampled = {r.id: t for r, t in zip(reqs, tokens)}
        done = sch.advance(plan, sampled)
        for r, t in zip(reqs, tokens):
            if r.finish_reason != "eos":
                self.stats.generated_tokens += 1
                if on_token:
                    on_token(r.id, t)
        for r in done:
            self.engine.end_request(r.id)
        return done

    def run(self, on_token: Optional[Callable[[Hashable, int], None]] = None) -> Dict[Hashable, Request]:
        while not self.scheduler.idle:
            self.step(on_token)
        return self.scheduler.finished


def generate(engine: Engine, prompts: Sequence[Sequence[int]], params=None, max_seqs: Optional[int] = None,
             max_step_tokens: int = DEFAULT_STEP_TOKENS) -> List[List[int]]:
    """The tokens generated after each prompt (lists of token ids); `params` is one SamplingParams or one per prompt."""
    if params is None:
        params = SamplingParams()
    per = list(params) if isinstance(params, (list, tuple)) else [params] * len(prompts)
    if len(per) != len(prompts):
        raise ValueError("generate: one SamplingParams per prompt, or one for all")
    gen = Generator(engine, max_seqs, max_step_tokens)
    for i, (p, sp) in enumerate(zip(prompts, per)):
        import copy
        gen.submit(Request(i, [int(t) for t in p], copy.copy(sp)))
    finished = gen.run()
    return [finished[i].generated for i in range(len(prompts))]
