"""Scheduler decisions on the CPU, no model.  The first tests restate the reference's
own vectors (tests/test_scheduler_edge_cases.py, tests/test_scheduler_invariants.py of
the reference), rescaled from page size 256 to 4."""

import random

import pytest

from tokensprint_amd.cache import CacheManager, GroupLayout, OutOfPages
from tokensprint_amd.config import SamplingParams
from tokensprint_amd.engine.request import Request, RequestStatus
from tokensprint_amd.engine.scheduler import Scheduler

P = 4


def make_scheduler(*, num_pages=8, budget=8, max_num_seqs=8, max_model_len=64, chunked=False,
                   windows=(None,)):
    groups = [GroupLayout(2, 16, w, (i,)) for i, w in enumerate(windows)]
    manager = CacheManager(groups, P, num_pages, max_num_seqs)
    return Scheduler(manager, max_num_batched_tokens=budget, max_num_seqs=max_num_seqs,
                     max_model_len=max_model_len, eos=-1, chunked_prefill=chunked)


def assert_queues(s):
    waiting = {r.ordinal for r in s.waiting}
    running = {r.ordinal for r in s.running}
    assert waiting.isdisjoint(running)
    assert all(r.status == RequestStatus.WAITING and r.cache is None for r in s.waiting)
    assert all(r.status == RequestStatus.RUNNING and r.cache is not None for r in s.running)
    s.manager.check()


def test_worked_example_of_chunked_prefill():
    """Prompt of 11, budget 8, page 4: portions 8 then 3, then single tokens; a page is
    taken exactly when a portion crosses into it."""
    s = make_scheduler(budget=8, chunked=True)
    req = Request(0, list(range(11)), SamplingParams(max_tokens=8))
    s.add_request(req)
    step = s.schedule()
    assert step == [req] and (req.num_cached_tokens, req.num_new_tokens) == (0, 8)
    assert len(req.block_table) == 2
    s.postprocess(step, [], [])
    assert (req.num_cached_tokens, req.num_new_tokens) == (8, 0)
    step = s.schedule()
    assert req.num_new_tokens == 3 and len(req.block_table) == 3
    s.postprocess(step, [100], [0])
    assert len(req) == 12 and req.num_cached_tokens == 11
    step = s.schedule()
    assert req.num_new_tokens == 1 and len(req.block_table) == 3      # 12th fits the tail
    s.postprocess(step, [101], [0])
    step = s.schedule()
    assert req.num_new_tokens == 1 and len(req.block_table) == 4      # 13th opens a page
    assert_queues(s)


def test_lone_request_that_cannot_grow_raises_out_of_pages():
    # the reference's generic "empty schedule" crash, here a named condition
    s = make_scheduler(num_pages=1, budget=64)
    req = Request(0, [1] * 3)
    s.add_request(req)
    step = s.schedule()
    s.postprocess(step, [2], [0])
    step = s.schedule()
    s.postprocess(step, [2], [0])
    with pytest.raises(OutOfPages, match="request 0 alone"):
        s.schedule()
    assert req.status == RequestStatus.RUNNING and req.cache is not None
    assert_queues(s)


def test_impossible_requests_are_refused_when_added():
    s = make_scheduler(num_pages=8, budget=8, chunked=False)
    with pytest.raises(ValueError, match="max_num_batched_tokens"):
        s.add_request(Request(0, [1] * 9))
    s = make_scheduler(num_pages=2, budget=64, chunked=True)
    with pytest.raises(ValueError, match="pages"):
        s.add_request(Request(0, [1] * 8))       # 8 tokens + 1 need 3 pages
    with pytest.raises(ValueError, match="max_model_len"):
        s.add_request(Request(0, [1] * 64))


def test_chunked_prefill_takes_the_budget():
    s = make_scheduler(num_pages=16, budget=5, chunked=True)
    req = Request(0, [1] * 20)
    s.add_request(req)
    assert s.schedule() == [req] and req.num_new_tokens == 5


def test_decode_proceeds_with_one_token_when_a_page_is_free():
    s = make_scheduler(num_pages=2, budget=64)
    req = Request(0, [1] * 4)
    s.add_request(req)
    s.postprocess(s.schedule(), [2], [0])
    step = s.schedule()
    assert step == [req] and req.num_new_tokens == 1


def test_admission_and_postprocess_invariants():
    s = make_scheduler(num_pages=16, budget=64)
    req = Request(0, [1] * 13)
    s.add_request(req)
    step = s.schedule()
    assert step == [req] and req.status == RequestStatus.RUNNING
    assert (req.num_cached_tokens, req.num_new_tokens) == (0, 13)
    assert len(req.block_table) == 4
    table = list(req.block_table)
    s.postprocess(step, [42], [0])
    assert (req.num_cached_tokens, req.num_new_tokens, len(req)) == (13, 0, 14)
    assert req.block_table == table
    assert_queues(s)


def test_finishing_frees_everything():
    s = make_scheduler()
    req = Request(0, [1] * 6, SamplingParams(max_tokens=1))
    s.add_request(req)
    s.postprocess(s.schedule(), [99], [0])
    assert req.status == RequestStatus.FINISHED and req.cache is None
    assert req not in s.running and req not in s.waiting
    assert s.manager.pools[0].num_used == 0 and s.manager.slots.num_free == 8
    assert s.is_finished()


def test_eos_stops_unless_ignored():
    s = make_scheduler()
    s.eos = 7
    a = Request(0, [1, 2], SamplingParams(max_tokens=5))
    b = Request(1, [1, 2], SamplingParams(max_tokens=5, ignore_eos=True))
    s.add_request(a); s.add_request(b)
    s.postprocess(s.schedule(), [7, 7], [0, 1])
    assert a.is_finished and not b.is_finished


def test_preemption_takes_the_last_running_request_to_the_front_of_waiting():
    s = make_scheduler(num_pages=4, budget=64)
    a, b, c = Request(0, [1] * 8), Request(1, [2] * 8), Request(2, [3] * 3)
    for r in (a, b, c):
        s.add_request(r)
    step = s.schedule()
    assert step == [a, b]                          # c does not fit: no skip-ahead
    s.postprocess(step, [5, 5], [0, 1])            # both at 9 tokens, pages full
    step = s.schedule()                            # a needs a page: b, the last, is preempted
    assert step == [a]
    assert b.status == RequestStatus.WAITING and s.waiting[0] is b and b.cache is None
    assert (b.num_cached_tokens, b.num_new_tokens, len(b)) == (0, 0, 9)   # tokens are kept
    assert b.num_preemptions == 1 and s.num_preemptions == 1
    assert_queues(s)
    # a step with a preemption admits nobody, although c would fit now
    assert c.status == RequestStatus.WAITING
    s.postprocess(step, [5], [0])
    a.max_tokens = 3
    step = s.schedule()
    s.postprocess(step, [5] * len(step), list(range(len(step))))
    assert a.is_finished
    step = s.schedule()                            # b comes back first, over all 9 tokens
    assert step[0] is b and b.num_new_tokens == 9


def test_recomputed_request_over_budget_runs_alone_when_not_chunked():
    s = make_scheduler(num_pages=8, budget=6, chunked=False)
    a = Request(0, [1] * 6, SamplingParams(max_tokens=8))
    s.add_request(a)
    s.postprocess(s.schedule(), [9], [0])
    s.running.remove(a)
    s.preempt(a)                                   # now 7 tokens to recompute, budget 6
    step = s.schedule()
    assert step == [a] and a.num_new_tokens == 7


def test_state_slots_bound_the_running_set():
    s = make_scheduler(num_pages=32, budget=64, max_num_seqs=2)
    reqs = [Request(i, [1] * 3) for i in range(3)]
    for r in reqs:
        s.add_request(r)
    assert s.schedule() == reqs[:2]
    assert {r.cache.slot for r in reqs[:2]} == {0, 1}


@pytest.mark.parametrize("seed", range(6))
def test_random_arrivals_with_a_tiny_pool_always_finish(seed):
    """Whatever the order, every request ends with exactly the tokens it would get with
    unlimited pages (tokens here are a function of the request and its length)."""
    rnd = random.Random(seed)
    s = make_scheduler(num_pages=rnd.choice([10, 14]), budget=rnd.choice([6, 16]),
                       max_num_seqs=4, max_model_len=40, chunked=True,
                       windows=(None, 5) if seed % 2 else (None,))
    pending = [Request(i, [rnd.randrange(50) for _ in range(rnd.randrange(1, 20))],
                       SamplingParams(max_tokens=rnd.randrange(1, 12))) for i in range(12)]
    everyone = list(pending)
    steps = 0
    while pending or not s.is_finished():
        while pending and rnd.random() < 0.5:
            s.add_request(pending.pop(0))
        if s.is_finished():
            continue
        step = s.schedule()
        assert sum(r.num_new_tokens for r in step) <= s.max_num_batched_tokens
        sampled = [i for i, r in enumerate(step)
                   if r.num_cached_tokens + r.num_new_tokens == len(r)]
        tokens = [(step[i].ordinal * 31 + len(step[i])) % 50 for i in sampled]
        s.postprocess(step, tokens, sampled)
        assert_queues(s)
        steps += 1
        assert steps < 5000
    for r in everyone:
        assert r.is_finished and r.num_completion_tokens == r.max_tokens
        n0 = r.num_prompt_tokens
        assert r.completion_token_ids == [(r.ordinal * 31 + n0 + i) % 50
                                          for i in range(r.max_tokens)]
    assert all(p.num_used == 0 for p in s.manager.pools)


# ------------------------------------------------------------------ prefix cache
def test_a_cached_prefix_is_not_computed_again():
    s = make_scheduler(num_pages=12, budget=32, chunked=True)
    s.manager.enable_prefix_cache()
    stem = list(range(1, 11))                          # two full pages and a half
    a = Request(0, stem + [40, 41], SamplingParams(max_tokens=2))
    s.add_request(a)
    assert s.schedule() == [a] and (a.num_cached_tokens, a.num_new_tokens) == (0, 12)
    s.postprocess([a], [7], [0])
    b = Request(1, stem + [50], SamplingParams(max_tokens=1))
    s.add_request(b)
    step = s.schedule()
    assert step == [a, b]
    assert (b.num_cached_tokens, b.num_new_tokens) == (8, 3)     # pages 0 and 1 shared
    assert b.cache.tables[0][:2] == a.cache.tables[0][:2]
    assert s.num_prefix_hit_tokens == 8
    assert sum(r.num_new_tokens for r in step) == 4
    s.postprocess(step, [8, 9], [0, 1])
    assert a.is_finished and b.is_finished
    assert s.manager.pools[0].num_used == 0
    # finished requests leave their full pages findable: prompt and first completion token
    c = Request(2, stem + [40, 41, 7, 8, 3], SamplingParams(max_tokens=1))
    s.add_request(c)
    s.schedule()
    assert c.num_cached_tokens == 12
    s.postprocess([c], [1], [0])
    assert_queues(s)


def test_a_prefix_hit_that_does_not_fit_leaves_nothing_behind():
    s = make_scheduler(num_pages=5, budget=32, chunked=True)
    s.manager.enable_prefix_cache()
    a = Request(0, list(range(1, 13)), SamplingParams(max_tokens=8))
    s.add_request(a)
    s.postprocess(s.schedule(), [5], [0])              # 3 pages full, a fourth for the decode
    s.postprocess(s.schedule(), [5], [0])
    b = Request(1, list(range(1, 13)) + [9, 9, 9, 9, 9], SamplingParams(max_tokens=1))
    s.add_request(b)                                   # shares 3 pages, needs 2 more: 1 free
    assert s.schedule() == [a]
    assert b.status == RequestStatus.WAITING and b.cache is None
    assert s.num_prefix_hit_tokens == 0
    assert [s.manager.pools[0].refs[p] for p in a.cache.tables[0]] == [1, 1, 1, 1]
    assert_queues(s)


@pytest.mark.parametrize("seed", range(4))
def test_random_arrivals_with_shared_prefixes_always_finish(seed):
    rnd = random.Random(100 + seed)
    s = make_scheduler(num_pages=rnd.choice([10, 14]), budget=rnd.choice([6, 16]),
                       max_num_seqs=4, max_model_len=40, chunked=bool(seed % 2))
    s.manager.enable_prefix_cache()
    stems = [[rnd.randrange(50) for _ in range(9)] for _ in range(2)]
    budget = s.max_num_batched_tokens
    pending = [Request(i, (rnd.choice(stems) + [rnd.randrange(50) for _ in range(rnd.randrange(1, 8))])[:budget],
                       SamplingParams(max_tokens=rnd.randrange(1, 12))) for i in range(12)]
    everyone = list(pending)
    steps = 0
    while pending or not s.is_finished():
        while pending and rnd.random() < 0.5:
            s.add_request(pending.pop(0))
        if s.is_finished():
            continue
        step = s.schedule()
        sampled = [i for i, r in enumerate(step)
                   if r.num_cached_tokens + r.num_new_tokens == len(r)]
        tokens = [(step[i].ordinal * 31 + len(step[i])) % 50 for i in sampled]
        s.postprocess(step, tokens, sampled)
        assert_queues(s)
        steps += 1
        assert steps < 5000
    for r in everyone:
        assert r.is_finished and r.num_completion_tokens == r.max_tokens
    assert s.num_prefix_hit_tokens > 0
    assert all(p.num_used == 0 for p in s.manager.pools)
