"""The scheduler's decisions, without a GPU: a stand-in for the engine reserves and commits what a step would write
and appends a token for every request that samples.  The first two tests hold the vectors of the reference's
tests/test_scheduler.py."""

import random

import pytest

from nanospec_amd.cache import CacheManager, GroupSpec, PoolExhausted
from nanospec_amd.engine.scheduler import Request, Scheduler
from nanospec_amd.sampling import SamplingParams


def manager(pages, page, slots=16):
    return CacheManager([GroupSpec("all")], pages, page, slots)


def req(i, n, max_tokens=4):
    return Request(i, list(range(n)), SamplingParams(max_tokens=max_tokens))


def run_step(s: Scheduler, token=1):
    """One engine step's worth of bookkeeping.  -> the work list."""
    work = s.next_batch()
    for w in work:
        w.sampled = w.samples  # as seen before any token is appended
        s.cache.reserve(w.req.id, w.n)
    for w in work:
        s.cache.commit(w.req.id, w.n)
        w.req.computed += w.n
    for w in work:
        if w.sampled:
            w.req.out_tokens.append(token)
            if len(w.req.out_tokens) >= w.req.params.max_tokens:
                s.finish(w.req)
    s.cache.check()
    return work


def ids(work):
    return [(w.req.id, w.n) for w in work]


def test_staggered_admission_and_decode_order():
    """reference tests/test_scheduler.py:9-22: one admission per step; a request is prefilled in the step it is admitted
    and decodes in the next; max_running caps."""
    s = Scheduler(manager(64, 4), max_admit=1)
    for i in range(3):
        s.add(req(i, 5, max_tokens=40))
    assert ids(run_step(s)) == [(0, 5)]
    assert ids(run_step(s)) == [(0, 1), (1, 5)]
    assert ids(run_step(s)) == [(0, 1), (1, 1), (2, 5)]
    assert [s.cache.get(r.id).length for r in s.running] == [7, 6, 5]
    s.max_running = 3
    s.add(req(3, 5))
    assert ids(run_step(s)) == [(0, 1), (1, 1), (2, 1)]  # the cap keeps request 3 waiting
    assert [r.id for r in s.waiting] == [3]


def test_admission_waits_for_pages_and_finish_frees():
    """reference tests/test_scheduler.py:25-42: admission reserves prompt + max_tokens; strictly first come first served."""
    m = manager(4, 4)
    s = Scheduler(m, max_admit=8)
    s.add(req(0, 12))  # 12 + 4 -> 4 pages
    s.add(req(1, 6))   # 6 + 4 -> 3 pages: does not fit beside request 0
    s.add(req(2, 1))   # 1 + 4 -> 2 pages: would fit, but may not overtake request 1
    s._admit()
    assert [r.id for r in s.running] == [0] and [r.id for r in s.waiting] == [1, 2]
    s.finish(s.running[0])
    assert m.num_free() == 4
    s._admit()
    assert [r.id for r in s.running] == [1]  # 3 pages spoken for, 1 left: request 2 (2 pages) waits
    s.finish(s.running[0])
    s._admit()
    assert [r.id for r in s.running] == [2]
    s.finish(s.running[0])
    assert not s.has_work and m.num_free() == 4
    m.check()


def test_a_request_that_can_never_fit_is_refused_at_once():
    s = Scheduler(manager(4, 4))
    with pytest.raises(PoolExhausted):
        s.add(req(0, 14, max_tokens=8))


def test_token_budget_cuts_prompts_into_portions():
    """Decoding requests come first with one token each; the rest of the budget goes to prompts in admission order,
    at most prefill_chunk per request; a request samples only in the step that ends its prompt."""
    s = Scheduler(manager(256, 4, slots=8), max_admit=8, max_step_tokens=16, prefill_chunk=10)
    s.add(req(0, 25, max_tokens=3))
    s.add(req(1, 7, max_tokens=3))
    w = run_step(s)
    assert ids(w) == [(0, 10), (1, 6)] and not any(x.sampled for x in w)
    w = run_step(s)
    assert ids(w) == [(0, 10), (1, 1)] and [x.sampled for x in w] == [False, True]
    w = run_step(s)
    assert ids(w) == [(0, 5), (1, 1)] and [x.sampled for x in w] == [True, True]  # request 1 decodes beside the last portion
    assert ids(run_step(s)) == [(0, 1), (1, 1)]
    assert [r.id for r in s.running] == [0]  # request 1 has its 3 tokens
    run_step(s)
    assert not s.has_work and s.cache.num_free() == 256


def test_budget_smaller_than_the_decoding_requests():
    """Nobody starves: with room for two of three decoding requests per step they take turns (the one that has waited
    longest goes first), so their outputs never differ by more than one token."""
    s = Scheduler(manager(64, 4), max_admit=8, max_step_tokens=2)
    reqs = [req(i, 1, max_tokens=5) for i in range(3)]
    for r in reqs:
        s.add(r)
    assert ids(run_step(s)) == [(0, 1), (1, 1)]
    assert ids(run_step(s)) == [(0, 1), (2, 1)]  # request 2 has waited longest, then request 0 by admission order
    assert ids(run_step(s)) == [(1, 1), (2, 1)]
    while s.has_work:
        assert sum(w.n for w in run_step(s)) <= 2
        live = [len(r.out_tokens) for r in reqs if r.state == "running"]
        assert not live or max(live) - min(live) <= 1
    assert all(len(r.out_tokens) == 5 for r in reqs)
    assert s.cache.num_free() == 64


def test_a_prompt_advances_although_the_decoding_requests_fill_the_budget():
    """Eight decoding requests and a budget of eight: an eighth of it (one token here) is kept for the oldest unfinished
    prompt, which would otherwise wait until a decoding request finishes; the decoding requests share what is left."""
    s = Scheduler(manager(256, 4), max_admit=16, max_step_tokens=8)
    dec = [req(i, 1, max_tokens=60) for i in range(8)]
    for r in dec:
        s.add(r)
    run_step(s)  # all eight have their one prompt token in the cache and decode from here on
    late = req(8, 30, max_tokens=2)
    s.add(late)
    for _ in range(29):
        work = run_step(s)
        assert sum(w.n for w in work) <= 8
        assert (8, 1) in ids(work)  # the prompt's token of this step
    assert late.computed == 29  # its last token left, it takes turns with the others like a decoding request
    for _ in range(4):
        run_step(s)
    assert late.state == "done" and len(late.out_tokens) == 2
    assert max(len(r.out_tokens) for r in dec) - min(len(r.out_tokens) for r in dec) <= 1
    # with a wider budget the prompt takes all that the decoding requests leave
    s2 = Scheduler(manager(256, 4), max_admit=16, max_step_tokens=20)
    for i in range(8):
        s2.add(req(i, 1, max_tokens=60))
    run_step(s2)
    s2.add(req(8, 30, max_tokens=2))
    assert ids(run_step(s2))[-1] == (8, 12)


def test_decoding_rows_count_as_the_engine_pads_them():
    """The engine rounds the rows of decoding requests up to a captured step's size and says so through ``decode_rows_cost``:
    the budget is charged for the padded rows where they fit it, so that such a step stays within it with its padding, and for
    the rows as they are where they do not."""
    buckets = (1, 2, 4, 8)
    cost = lambda n: next((b for b in buckets if b >= n), n) if n else 0
    s = Scheduler(manager(256, 4), max_admit=16, max_step_tokens=32)
    s.decode_rows_cost = cost
    for i in range(5):
        s.add(req(i, 1, max_tokens=40))
    run_step(s)
    s.add(req(5, 100, max_tokens=2))
    work = run_step(s)
    assert ids(work) == [(i, 1) for i in range(5)] + [(5, 24)]  # five rows are padded to eight: 24 of 32 are left
    # a budget of six: five rows padded to eight do not fit, so they are charged as the five they are (nobody who fits is
    # left out because of padding) and the prompt has the one token that is left
    s = Scheduler(manager(256, 4), max_admit=16, max_step_tokens=6)
    s.decode_rows_cost = cost
    for i in range(5):
        s.add(req(i, 1, max_tokens=40))
    run_step(s)
    s.add(req(5, 100, max_tokens=2))
    for _ in range(6):
        assert ids(run_step(s)) == [(i, 1) for i in range(5)] + [(5, 1)]
    # a budget that is no multiple of the padding: 20 decoding requests under 24 all advance (32 padded rows do not fit),
    # where a budget of 40 charges the 32 and leaves a prompt 8
    for budget, portion in ((24, 4), (40, 8)):
        s = Scheduler(manager(1024, 4, slots=32), max_admit=32, max_step_tokens=budget)
        s.decode_rows_cost = lambda n: next((b for b in (1, 2, 4, 8, 16, 32) if b >= n), n) if n else 0
        for i in range(20):
            s.add(req(i, 1, max_tokens=40))
        run_step(s)
        s.add(req(20, 100, max_tokens=2))
        assert ids(run_step(s)) == [(i, 1) for i in range(20)] + [(20, portion)]


def test_preemption_when_pages_run_out():
    """Under "preempt" admission needs only the first portion.  When a step does not fit, the request admitted last goes
    back to the HEAD of the queue with its output kept; later it is recomputed from prompt + output."""
    m = manager(6, 4)
    s = Scheduler(m, max_admit=8, on_exhaustion="preempt")
    a, b = req(0, 8, max_tokens=12), req(1, 8, max_tokens=12)
    s.add(a), s.add(b)
    assert ids(run_step(s)) == [(0, 8), (1, 8)]  # 2 + 2 pages
    for _ in range(4):
        assert ids(run_step(s)) == [(0, 1), (1, 1)]  # 12 tokens each: 3 + 3 pages, pool full
    w = run_step(s)  # token 13 of each needs a 4th page: only request 0 keeps running
    assert ids(w) == [(0, 1)] and b.state == "waiting" and b.preemptions == 1 and s.waiting[0] is b
    assert len(b.out_tokens) == 5 and b.computed == 0
    m.check()
    while a.state != "done":
        run_step(s)
    w = run_step(s)
    assert ids(w) == [(1, 13)] and w[0].sampled  # recomputed from prompt + the 5 tokens it had
    while s.has_work:
        run_step(s)
    assert len(a.out_tokens) == len(b.out_tokens) == 12 and m.num_free() == 6
    # alone and still too long for what is left of the pool: an error, not an endless loop
    s2 = Scheduler(manager(2, 4), on_exhaustion="preempt")
    s2.add(Request(0, list(range(4)), SamplingParams(max_tokens=4)))
    s2.cache.admit("someone else"), s2.cache.reserve("someone else", 1)
    run_step(s2)
    with pytest.raises(PoolExhausted):
        run_step(s2)


def test_reserve_policy_never_runs_out():
    rng = random.Random(3)
    m = manager(40, 4, slots=8)
    s = Scheduler(m, max_admit=3, max_running=7, max_step_tokens=24, prefill_chunk=9)
    reqs = [Request(i, list(range(rng.randint(1, 30))), SamplingParams(max_tokens=rng.randint(1, 20))) for i in range(40)]
    for r in reqs:
        s.add(r)
    steps = 0
    while s.has_work:
        work = run_step(s)
        assert work and sum(w.n for w in work) <= 24
        steps += 1
        assert steps < 2000
    assert all(r.state == "done" and len(r.out_tokens) == r.params.max_tokens for r in reqs)
    assert m.num_free() == 40 and s.preempted_total == 0


@pytest.mark.parametrize("seed", range(4))
def test_preempt_policy_always_finishes(seed):
    rng = random.Random(seed)
    m = manager(24, 4, slots=8)
    s = Scheduler(m, max_admit=4, max_running=6, max_step_tokens=32, prefill_chunk=16, on_exhaustion="preempt")
    reqs = [Request(i, list(range(rng.randint(1, 20))), SamplingParams(max_tokens=rng.randint(1, 30))) for i in range(25)]
    for r in reqs:
        s.add(r)
    steps = 0
    while s.has_work:
        run_step(s)
        steps += 1
        assert steps < 5000
    assert all(r.state == "done" and len(r.out_tokens) == r.params.max_tokens for r in reqs)
    assert m.num_free() == 24 and s.preempted_total > 0
