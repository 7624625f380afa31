"""The generator's bookkeeping around a failing step, with an engine that computes nothing."""

import pytest
import torch

from llmx_amd.cache import CacheManager, GroupSpec
from llmx_amd.engine.generation import Generator
from llmx_amd.engine.scheduler import Request
from llmx_amd.sampling import SamplingParams


class _Spec:
    eos_token_id = None


class _FailingEngine:
    """What Generator reads of an engine; its second step raises."""

    def __init__(self):
        self.cache = CacheManager([GroupSpec("kv", 4, 32)], max_requests=2)
        self.max_requests, self.max_positions, self.vocab_size = 2, 128, 50
        self.device = torch.device("cpu")
        self.spec = _Spec()
        self.steps = 0

    def add_request(self, rid):
        return self.cache.open(rid)

    def end_request(self, rid):
        self.cache.close(rid)

    def has_request(self, rid):
        return self.cache.is_open(rid)

    def step(self, entries):
        self.steps += 1
        if self.steps == 2:
            raise RuntimeError("the step failed")
        for e in entries:
            self.cache.prepare(e.request, len(e.tokens))
            self.cache.commit(e.request)
        return torch.zeros((0, self.vocab_size))


def test_a_failing_round_leaves_no_request_open():
    eng = _FailingEngine()
    gen = Generator(eng, max_seqs=2, max_step_tokens=4)
    gen.submit(Request(0, list(range(10)), SamplingParams(max_tokens=2, temp=0.0)))
    gen.submit(Request(1, list(range(6)), SamplingParams(max_tokens=2, temp=0.0)))
    gen.step()
    assert eng.cache.pages_in_use() > 0
    with pytest.raises(RuntimeError, match="the step failed"):
        gen.step()
    assert eng.cache.pages_in_use() == 0 and eng.cache.slots.in_use == 0 and eng.cache.live() == []
    # the scheduler retired them too: reservations returned, nothing running, both finished with reason "error"
    sch = gen.scheduler
    assert sch.reserved == [0] and sch.idle and not sch.running
    assert {r.finish_reason for r in sch.finished.values()} == {"error"} and set(sch.finished) == {0, 1}
    # the scheduler goes on: a request submitted after the failure finds every seat and page free
    gen.submit(Request(2, list(range(5)), SamplingParams(max_tokens=1, temp=0.0)))
    assert [r.id for r in sch.admit()] == [2]
