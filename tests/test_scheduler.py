"""The scheduler's decisions, without a model: a simulated executor feeds it tokens
(the reference tests its policy the same way: /root/reference/docs/TESTS.md:829)."""

import random

import pytest

from llmx_amd.cache import CacheManager, GroupSpec
from llmx_amd.engine.scheduler import Request, Scheduler, SchedulerError
from llmx_amd.sampling import SamplingParams

EOS = 99


def run(s, token_for=lambda r, i: 7, max_rounds=10000, cache=None):
    """Plays the scheduler against a simulated executor; returns the list of plans."""
    plans = []
    while not s.idle:
        for r in s.admit():
            if cache:
                cache.open(r.id)
        plan = s.plan()
        assert plan, "an empty round with requests left"
        by_id = {r.id: r for r in s.running}
        if cache:
            for e in plan:
                cache.prepare(e.request, len(e.tokens))     # must never raise: admission reserved the pages
                cache.commit(e.request)
        sampled = {e.request: token_for(by_id[e.request], len(by_id[e.request].generated)) for e in plan if e.wants_logits}
        done = s.advance(plan, sampled)
        if cache:
            for r in done:
                cache.close(r.id)
        plans.append(plan)
        assert len(plans) < max_rounds
    return plans


def greedy(n):
    return SamplingParams(max_tokens=n, temp=0.0)


def test_portions_budget_and_decode_first():
    s = Scheduler([GroupSpec("kv", 4, 100)], max_seqs=4, max_step_tokens=8, eos_token_id=EOS)
    s.submit(Request("a", list(range(10)), greedy(3)))
    s.submit(Request("b", list(range(5)), greedy(2)))
    plans = run(s)
    shape = [[(e.request, len(e.tokens), e.wants_logits) for e in p] for p in plans]
    assert shape[0] == [("a", 8, False)]                                   # the budget cuts the prompt
    assert shape[1] == [("a", 2, True), ("b", 5, True)]                    # the portion reaching the end wants logits
    assert shape[2] == [("a", 1, True), ("b", 1, True)]                    # decoding, in order of admission
    assert all(sum(len(e.tokens) for e in p) <= 8 for p in plans)
    assert s.finished["a"].generated == [7, 7, 7] and s.finished["a"].finish_reason == "length"
    assert s.finished["b"].generated == [7, 7]
    # the decoded token fed is the one sampled before
    assert plans[2][0].tokens == [7]
    # decoding requests come before prompt portions
    s = Scheduler([GroupSpec("kv", 4, 100)], max_seqs=4, max_step_tokens=6)
    s.submit(Request("a", [1, 2], greedy(5)))
    run_one = lambda: (s.admit(), s.plan())[1]
    p = run_one()
    s.advance(p, {"a": 3})
    s.submit(Request("b", list(range(20)), greedy(2)))
    p = run_one()
    assert [(e.request, len(e.tokens)) for e in p] == [("a", 1), ("b", 5)]


def test_eos_and_ignore_eos():
    s = Scheduler([GroupSpec("kv", 4, 100)], 2, 16, eos_token_id=EOS)
    s.submit(Request("a", [1, 2, 3], greedy(10)))
    s.submit(Request("b", [1, 2, 3], SamplingParams(max_tokens=4, temp=0.0, ignore_eos=True)))
    run(s, token_for=lambda r, i: EOS if i == 2 else 5)
    assert s.finished["a"].generated == [5, 5] and s.finished["a"].finish_reason == "eos"       # the end token is not kept
    assert s.finished["b"].generated == [5, 5, EOS, 5] and s.finished["b"].finish_reason == "length"


def test_stop_sequences():
    """Generation ends when the generated ids end with a stop sequence; the completing token is kept (the reference
    keeps the token that completes its stop text and does not feed it: /root/reference/src/inference/generate.hpp:29-36)."""
    s = Scheduler([GroupSpec("kv", 4, 100)], 3, 16, eos_token_id=EOS)
    seq = [5, 6, 7, 6, 7, 8, 9]
    s.submit(Request("one", [1, 2], SamplingParams(max_tokens=7, temp=0.0, stop=(7, 8))))
    s.submit(Request("two", [1, 2], SamplingParams(max_tokens=7, temp=0.0, stop=((9, 9), (6, 7, 6)))))
    s.submit(Request("none", [1, 2], SamplingParams(max_tokens=7, temp=0.0, stop=((8, 7),))))
    plans = run(s, token_for=lambda r, i: seq[i])
    assert s.finished["one"].generated == [5, 6, 7, 6, 7, 8] and s.finished["one"].finish_reason == "stop"
    assert s.finished["two"].generated == [5, 6, 7, 6] and s.finished["two"].finish_reason == "stop"
    assert s.finished["none"].generated == seq and s.finished["none"].finish_reason == "length"
    # the completing token is never fed: after the step that drew it the request is gone
    assert all(e.request != "two" for p in plans[4:] for e in p)
    assert s.reserved == [0]
    assert SamplingParams(stop=()).validate().stop == ()
    for bad in (((),), tuple(range(300)), ((1,),) * 17, (-1,)):
        with pytest.raises(ValueError, match="stop"):
            SamplingParams(stop=bad).validate()


def test_fifo_admission_and_reservation():
    """Pages run out: a request waits in the queue until running ones finish; nobody overtakes the head of the queue;
    a running request never fails to get a page (the cache manager is driven alongside and never raises)."""
    groups = [GroupSpec("kv", 4, 12)]
    cache = CacheManager(groups, max_requests=3)
    s = Scheduler(groups, max_seqs=3, max_step_tokens=16)
    s.submit(Request("a", list(range(20)), greedy(4)))      # 6 pages
    s.submit(Request("b", list(range(18)), greedy(6)))      # 6 pages
    s.submit(Request("c", list(range(30)), greedy(2)))      # 8 pages: must wait for both
    s.submit(Request("d", [1], greedy(1)))                  # 1 page: would fit, but may not overtake c
    plans = run(s, cache=cache)
    first_seen = {}
    for i, p in enumerate(plans):
        for e in p:
            first_seen.setdefault(e.request, i)
    last_a = max(i for i, p in enumerate(plans) for e in p if e.request == "a")
    last_b = max(i for i, p in enumerate(plans) for e in p if e.request == "b")
    assert first_seen["c"] > max(last_a, last_b)
    assert first_seen["d"] >= first_seen["c"]
    assert cache.pages_in_use() == 0 and s.reserved == [0]
    assert [s.finished[k].order for k in "abcd"] == [0, 1, 2, 3]


def test_requests_that_can_never_fit_are_refused_at_submit():
    s = Scheduler([GroupSpec("kv", 4, 10)], 2, 16, max_positions=64)
    with pytest.raises(SchedulerError, match="needs 11 pages of kv, the cache holds 10"):
        s.submit(Request("big", list(range(40)), greedy(4)))
    with pytest.raises(SchedulerError, match="needs 70 positions"):
        Scheduler([GroupSpec("kv", 4, 100)], 2, 16, max_positions=64).submit(Request("long", list(range(60)), greedy(10)))
    with pytest.raises(SchedulerError, match="empty prompt"):
        s.submit(Request("e", [], greedy(1)))
    s.submit(Request("ok", [1], greedy(1)))
    with pytest.raises(SchedulerError, match="already submitted"):
        s.submit(Request("ok", [1], greedy(1)))
    with pytest.raises(ValueError, match="top_p"):
        s.submit(Request("p", [1], SamplingParams(top_k=0, top_p=1.5)))


def test_windowed_groups_reserve_a_window_not_the_whole_request():
    groups = [GroupSpec("all", 4, 1000), GroupSpec("win", 4, 12, window=8)]
    s = Scheduler(groups, 2, max_step_tokens=16)
    s.submit(Request("a", list(range(300)), greedy(50)))     # 88 pages of "all", but only (8+16)/4+1 = 7 of "win"
    s.admit()
    assert s.reserved == [88, 7]


@pytest.mark.parametrize("seed", range(5))
def test_random_loads_finish_and_return_everything(seed):
    rng = random.Random(seed)
    groups = [GroupSpec("kv", 8, 60)]
    cache = CacheManager(groups, max_requests=4)
    s = Scheduler(groups, max_seqs=4, max_step_tokens=rng.choice([4, 16, 64]), eos_token_id=EOS)
    wanted = {}
    for i in range(25):
        n_prompt, n_new = rng.randint(1, 120), rng.randint(1, 40)
        s.submit(Request(i, [rng.randrange(90) for _ in range(n_prompt)], greedy(n_new)))
        wanted[i] = n_new
    plans = run(s, token_for=lambda r, i: (r.id * 31 + i) % 90, cache=cache)
    for i, n_new in wanted.items():
        assert s.finished[i].generated == [(i * 31 + j) % 90 for j in range(n_new)]   # its tokens are those of its run alone
    assert cache.pages_in_use() == 0 and cache.slots.in_use == 0 and s.reserved == [0]
    assert all(len({e.request for e in p}) == len(p) for p in plans)                     # a request at most once a step
    assert all(sum(len(e.tokens) for e in p) <= s.max_step_tokens for p in plans)


def test_the_last_token_the_limit_allows_is_fed_without_logits():
    """At max_tokens the last token goes into the cache in the next step (no logits wanted) and then the request ends;
    an end token and a token completing a stop sequence are never fed (/root/reference/src/inference/generate.hpp:28-45)."""
    groups = [GroupSpec("kv", 4, 100)]
    cache = CacheManager(groups, max_requests=3)
    s = Scheduler(groups, 3, 16, eos_token_id=EOS)
    s.submit(Request("len", [1, 2, 3], greedy(2)))
    s.submit(Request("eos", [1, 2, 3], greedy(5)))
    s.submit(Request("stop", [1, 2, 3], SamplingParams(max_tokens=5, temp=0.0, stop=(5, 5))))
    held = {}

    def token_for(r, i):
        return EOS if (r.id == "eos" and i == 1) else 5

    plans = []
    while not s.idle:
        for r in s.admit():
            cache.open(r.id)
        plan = s.plan()
        by_id = {r.id: r for r in s.running}
        for e in plan:
            cache.prepare(e.request, len(e.tokens))
            cache.commit(e.request)
        done = s.advance(plan, {e.request: token_for(by_id[e.request], len(by_id[e.request].generated)) for e in plan if e.wants_logits})
        for r in done:
            held[r.id] = cache.length(r.id)
            cache.close(r.id)
        plans.append([(e.request, list(e.tokens), e.wants_logits) for e in plan])
    assert plans[2] == [("len", [5], False)]                 # step 0: prompts, step 1: second tokens, step 2: the fed last token
    assert s.finished["len"].generated == [5, 5] and held["len"] == 3 + 2       # the cache held the whole reply
    assert s.finished["eos"].generated == [5] and held["eos"] == 3 + 1          # the end token was neither kept nor fed
    assert s.finished["stop"].generated == [5, 5] and held["stop"] == 3 + 1     # the completing token was kept, not fed
    assert s.reserved == [0] and cache.pages_in_use() == 0
    # without the feed the request ends with the step that drew its last token
    s = Scheduler(groups, 1, 16, feed_last=False)
    s.submit(Request("a", [1, 2, 3], greedy(2)))
    assert len(run(s)) == 2
