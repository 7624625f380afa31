"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes, finishes and frees.

Policy (decisions only; it owns no model and is tested with a simulated executor):
  * Admission is first come, first served.  A request is admitted while a seat is free and every cache group can
    reserve the pages it will hold at its largest (prompt + max_tokens, or a window's worth): a running request
    therefore never runs out of pages.  A request that could not fit even alone is refused when submitted.  When the
    head of the queue does not fit, admission stops (no overtaking) until running requests finish and free pages.
  * A step takes the decoding requests first, one token each, in order of admission, then portions of prompts in order
    of admission while the step's token budget lasts; a portion wants logits only when it reaches the prompt's end.
  * A request finishes on its end token (not kept, unless ignore_eos), when its generated ids end with one of its
    stop sequences, or at max_tokens; its pages and slot go back at once.  The last token that max_tokens allows is
    fed in the next step, without logits, before the request ends, so that what the cache holds is the whole reply
    (/root/reference/src/inference/generate.hpp:28-45: an end token and the token completing a stop text are not fed,
    the last token the limit allows is); `feed_last=False` skips that step.
The shape follows the reference's scheduler (/root/reference/src/server/scheduler.hpp:1187-1376 form, :752-766 admission,
:2514-2571 retire; reservation: /root/reference/src/server/policy.hpp:153-158).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional, Sequence

from ..cache.manager import GroupSpec
from ..sampling.params import SamplingParams, XorShift64

DEFAULT_STEP_TOKENS = 512   # the reference's default prompt batch (runtime.hpp:401, --ubatch)


class SchedulerError(ValueError):
    pass


@dataclass
class Request:
    id: Hashable
    prompt: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    generated: List[int] = field(default_factory=list)
    fed: int = 0                       # tokens of prompt + generated already in the cache
    state: str = "waiting"             # waiting | running | finished
    finish_reason: Optional[str] = None  # "eos" | "stop" | "length" | "error"
    reserved: List[int] = field(default_factory=list)
    rng: XorShift64 = None
    order: int = -1                    # order of admission

    def __post_init__(self):
        if self.rng is None:
            self.rng = XorShift64(self.params.seed)

    @property
    def decoding(self) -> bool:
        """Its prompt is in the cache and its last sampled token is the one token not yet fed."""
        return self.state == "running" and len(self.generated) > 0 and self.fed == len(self.prompt) + len(self.generated) - 1

    @property
    def prompt_left(self) -> int:
        return max(0, len(self.prompt) - self.fed)


@dataclass(frozen=True)
class PlannedEntry:
    request: Hashable
    tokens: List[int]
    wants_logits: bool


class Scheduler:
    def __init__(self, groups: Sequence[GroupSpec], max_seqs: int, max_step_tokens: int = DEFAULT_STEP_TOKENS,
                 max_positions: Optional[int] = None, eos_token_id: Optional[int] = None, feed_last: bool = True):
        if max_seqs < 1 or max_step_tokens < 1:
            raise SchedulerError("scheduler: max_seqs and max_step_tokens must be at least 1")
        self.groups = list(groups)
        self.max_seqs = max_seqs
        self.max_step_tokens = max_step_tokens
        self.max_positions = max_positions
        self.eos = eos_token_id
        self.feed_last = bool(feed_last)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: Dict[Hashable, Request] = {}
        self.reserved = [0] * len(self.groups)
        self._admitted = 0
        self._ids = set()

    # -- submitting -------------------------------------------------------------
    def _need(self, r: Request) -> List[int]:
        total = len(r.prompt) + r.params.max_tokens
        return [g.peak_pages(total, self.max_step_tokens) for g in self.groups]

    def submit(self, request: Request) -> None:
        if request.id in self._ids:
            raise SchedulerError(f"scheduler: request {request.id!r} was already submitted")
        if not request.prompt:
            raise SchedulerError("scheduler: empty prompt")
        request.params.validate()
        total = len(request.prompt) + request.params.max_tokens
        if self.max_positions is not None and total > self.max_positions:
            raise SchedulerError(f"scheduler: request {request.id!r} needs {total} positions, the engine reaches {self.max_positions}")
        for g, need in zip(self.groups, self._need(request)):
            if need > g.n_pages:
                raise SchedulerError(f"scheduler: request {request.id!r} needs {need} pages of {g.name}, the cache holds {g.n_pages}")
        self._ids.add(request.id)
        self.waiting.append(request)

    # -- one round ----------------------------------------------------------------
    def admit(self) -> List[Request]:
        """Moves requests from the queue to the running set while seats and reservations allow; returns the newly admitted."""
        new = []
        while self.waiting and len(self.running) < self.max_seqs:
            r = self.waiting[0]
            need = self._need(r)
            if any(self.reserved[i] + need[i] > g.n_pages for i, g in enumerate(self.groups)):
                break
            self.waiting.popleft()
            for i, n in enumerate(need):
                self.reserved[i] += n
            r.reserved = need
            r.state = "running"
            r.order = self._admitted
            self._admitted += 1
            self.running.append(r)
            new.append(r)
        return new

    def plan(self) -> List[PlannedEntry]:
        """The next step's batch: decoding requests first, then prompt portions under the token budget."""
        budget = self.max_step_tokens
        entries: List[PlannedEntry] = []
        for r in self.running:
            if r.decoding and budget > 0:
                # a request that reached max_tokens feeds its last token and wants nothing more
                entries.append(PlannedEntry(r.id, [r.generated[-1]], r.finish_reason is None))
                budget -= 1
        for r in self.running:
            if budget <= 0:
                break
            left = r.prompt_left
            if left > 0:
                n = min(left, budget)
                entries.append(PlannedEntry(r.id, r.prompt[r.fed:r.fed + n], n == left))
                budget -= n
        return entries

    def advance(self, entries: Sequence[PlannedEntry], sampled: Dict[Hashable, int]) -> List[Request]:
        """Records that `entries` ran and which token each wanting request drew; returns the requests that finished."""
        by_id = {r.id: r for r in self.running}
        done = []
        for e in entries:
            r = by_id[e.request]
            r.fed += len(e.tokens)
            if not e.wants_logits:
                if r.finish_reason is not None:      # its last token is in the cache now
                    done.append(r)
                continue
            tok = sampled[e.request]
            if self.eos is not None and tok == self.eos and not r.params.ignore_eos:
                r.finish_reason = "eos"
            else:
                r.generated.append(tok)
                if any(len(r.generated) >= len(s) and tuple(r.generated[-len(s):]) == s for s in r.params.stop):
                    r.finish_reason = "stop"       # the token that completes a stop sequence is kept and not fed
                elif len(r.generated) >= r.params.max_tokens:
                    r.finish_reason = "length"
            if r.finish_reason and not (r.finish_reason == "length" and self.feed_last):
                done.append(r)
        for r in done:
            self.running.remove(r)
            for i, n in enumerate(r.reserved):
                self.reserved[i] -= n
            r.state = "finished"
            self.finished[r.id] = r
        return done

    def fail_running(self) -> List[Request]:
        """The round failed: every running request is retired with finish reason "error" and its reservation returned;
        requests that wait stay in the queue.  Returns the retired requests."""
        failed = list(self.running)
        for r in failed:
            for i, n in enumerate(r.reserved):
                self.reserved[i] -= n
            r.reserved = []
            r.state = "finished"
            r.finish_reason = "error"
            self.finished[r.id] = r
        self.running.clear()
        return failed

    @property
    def idle(self) -> bool:
        return not self.waiting and not self.running
