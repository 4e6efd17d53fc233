"""The scheduler's decisions, on the CPU, with a cache manager that holds no
device memory and a stand-in for the model that 'samples' a counter."""

import random

import pytest

from zig_ai_amd.cache import CacheManager, OutOfPages
from zig_ai_amd.engine.scheduler import FINISHED, Request, Scheduler
from zig_ai_amd.parts import PagedNeed, StateNeed


def make(num_pages=16, page_size=4, num_slots=4, **kw):
    cache = CacheManager({0: StateNeed((4, 3)), 1: PagedNeed.kv(1, 16)}, page_size, num_pages,
                         num_slots, allocate=False)
    return cache, Scheduler(cache, **kw)


def drive(cache, sched, max_steps=10000, on_plan=None):
    """Run to completion the way the engine does: reserve, 'compute', commit, update."""
    steps = []
    while sched.has_work():
        plan = sched.schedule()
        assert plan, "work is left but nothing was scheduled"
        if on_plan:
            on_plan(plan)
        for e in plan:
            cache.reserve(e.request.id, e.count)
        for e in plan:
            assert e.start == cache.num_tokens(e.request.id) == e.request.num_computed
            cache.commit(e.request.id, e.count)
        sampled = {e.request.id: 1000 + len(e.request.output) for e in plan if e.samples}
        sched.update(plan, sampled)
        cache.check()
        steps.append(plan)
        assert len(steps) < max_steps
    return steps


def test_admission_gives_a_non_empty_batch():
    """/root/reference/tests/test_paged_attention.zig:222-237."""
    cache, sched = make()
    sched.add(Request("a", [1, 2, 3], 2))
    plan = sched.schedule()
    assert len(plan) == 1 and plan[0].count == 3 and plan[0].samples


def test_budget_and_portions():
    cache, sched = make(num_pages=64, max_num_batched_tokens=10, chunk_size=6)
    sched.add(Request("a", list(range(20)), 3))
    sched.add(Request("b", list(range(4)), 3))
    seen = []
    steps = drive(cache, sched, on_plan=lambda p: seen.append([(e.request.id, e.start, e.count) for e in p]))
    for plan in steps:
        assert sum(e.count for e in plan) <= 10
        assert all(e.count <= 6 for e in plan)
    assert seen[0] == [("a", 0, 6), ("b", 0, 4)]       # FIFO; the budget is shared
    assert seen[1][0] == ("b", 4, 1)                     # decoding requests are served first
    assert seen[1][1] == ("a", 6, 6)
    # a's prompt is cut 6, 6, 6, 2; only the step that reaches its last token samples
    a_entries = [(e.start, e.count, e.samples) for plan in steps for e in plan if e.request.id == "a"]
    assert a_entries[:4] == [(0, 6, False), (6, 6, False), (12, 6, False), (18, 2, True)]
    for r in sched.finished:
        assert r.output == [1000, 1001, 1002] and r.finish_reason == "length"
    assert all(g.pool.free_count == g.pool.size for g in cache.groups)
    assert cache.slots.free_count == cache.slots.size


def test_portions_down_to_one_token():
    cache, sched = make(num_pages=64, max_num_batched_tokens=3, chunk_size=2)
    sched.add(Request("a", list(range(7)), 2))
    steps = drive(cache, sched)
    assert [e.count for p in steps for e in p][:4] == [2, 2, 2, 1]


def test_max_num_seqs_and_slots_limit_admission():
    cache, sched = make(num_pages=64, num_slots=2, max_num_seqs=8)
    for i in range(4):
        sched.add(Request(i, [1, 2], 2))
    plan = sched.schedule()
    assert [e.request.id for e in plan] == [0, 1]        # two slots only
    cache2, sched2 = make(num_pages=64, num_slots=4, max_num_seqs=1)
    for i in range(3):
        sched2.add(Request(i, [1, 2], 2))
    assert [e.request.id for e in sched2.schedule()] == [0]


def test_head_of_line_is_not_overtaken():
    cache, sched = make(num_pages=4, page_size=4, chunk_size=64, max_num_batched_tokens=64)
    sched.add(Request("a", list(range(8)), 1))      # 2 pages
    sched.add(Request("big", list(range(12)), 1))   # 3 pages: does not fit beside a
    sched.add(Request("small", [1], 1))             # would fit, but must wait its turn
    plan = sched.schedule()
    assert [e.request.id for e in plan] == ["a"]


def test_eos_and_length():
    cache, sched = make()
    r = Request("a", [1, 2], 5, eos_token_id=1001)
    sched.add(r)
    drive(cache, sched)
    assert r.output == [1000, 1001] and r.finish_reason == "eos" and r.phase == FINISHED
    z = Request("z", [1], 0)
    sched.add(z)
    assert z.phase == FINISHED and not sched.has_work()
    with pytest.raises(ValueError):
        sched.add(Request("e", [], 3))


def test_pages_run_out_preempts_the_latest_and_recomputes():
    """A pool of 4 pages: the second request is preempted when the first needs a
    page, and comes back after the first has finished (the scenario of
    /root/reference/tests/test_paged_attention.zig:307-341, with recomputation
    instead of a host copy)."""
    cache, sched = make(num_pages=4, page_size=4, chunk_size=64, max_num_batched_tokens=64)
    a = Request("a", list(range(8)), 6)     # 2 pages, a third at its 1st new token... 9th token
    b = Request("b", list(range(7)), 6)     # 2 pages
    sched.add(a)
    sched.add(b)
    log = []
    drive(cache, sched, on_plan=lambda p: log.append([(e.request.id, e.start, e.count) for e in p]))
    assert b.preemptions >= 1 and a.preemptions == 0
    assert sched.preemption_count == b.preemptions
    # nothing lost, nothing duplicated
    assert a.output == [1000 + i for i in range(6)]
    assert b.output == [1000 + i for i in range(6)]
    # after the preemption b ran its prompt plus what it had generated, from position 0
    restart = [entry for plan in log for entry in plan if entry[0] == "b" and entry[1] == 0]
    assert len(restart) == 1 + b.preemptions
    assert restart[-1][2] > 7 or b.preemptions == 0
    assert all(g.pool.free_count == g.pool.size for g in cache.groups)


def test_request_that_cannot_fit_alone_raises():
    cache, sched = make(num_pages=2, page_size=4, chunk_size=64, max_num_batched_tokens=64)
    sched.add(Request("huge", list(range(9)), 1))
    with pytest.raises(OutOfPages, match="whole pool"):
        sched.schedule()
    cache, sched = make(num_pages=2, page_size=4)
    sched.add(Request("grows", list(range(8)), 4))
    with pytest.raises(OutOfPages, match="whole pool"):
        drive(cache, sched)


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_finish_in_order_of_fairness(seed):
    rng = random.Random(seed)
    cache, sched = make(num_pages=rng.choice([12, 20, 40]), page_size=4, num_slots=rng.choice([2, 4]),
                        max_num_seqs=4, max_num_batched_tokens=rng.choice([8, 16, 64]),
                        chunk_size=rng.choice([3, 8, 32]))
    reqs = []
    for i in range(12):
        r = Request(i, [rng.randrange(50) for _ in range(rng.randint(1, 20))], rng.randint(1, 12))
        reqs.append(r)
        sched.add(r)
    drive(cache, sched)
    for r in reqs:
        assert r.phase == FINISHED
        assert r.output == [1000 + k for k in range(r.max_new_tokens)]   # none lost or doubled
    assert all(g.pool.free_count == g.pool.size for g in cache.groups)
    assert cache.slots.free_count == cache.slots.size


SEEDS = range(30)


def run_differential(seed):
    """One random workload through the host library and through the plain statement
    of the policy (tests/plain_scheduler.py) in lockstep; returns what happened."""
    from plain_scheduler import FREED, PlainCache, PlainOutOfPages, PlainScheduler
    seen = {"preemptions": 0, "refused": 0, "freed": 0, "steps": 0, "eos": 0}
    rng = random.Random(seed)
    page_size = rng.choice([2, 4, 8])
    windows = [0] + ([rng.choice([5, 9, 16])] if seed % 2 else [])
    num_slots = rng.randint(2, 5)
    num_pages = rng.randint(4, 11)
    limits = dict(max_num_seqs=rng.randint(1, 5), max_num_batched_tokens=rng.randint(3, 24),
                  chunk_size=rng.randint(2, 12), max_model_len=rng.choice([0, 0, 30]))
    needs = {0: StateNeed((4, 3))}
    for g, w in enumerate(windows):
        needs[1 + g] = PagedNeed.kv(1, 16, w)
    cache = CacheManager(needs, page_size, num_pages, num_slots, allocate=False)
    sched = Scheduler(cache, **limits)
    pcache = PlainCache(windows, num_pages, page_size, num_slots)
    psched = PlainScheduler(pcache, limits["max_num_seqs"], limits["max_num_batched_tokens"],
                            limits["chunk_size"], limits["max_model_len"])
    biggest = (num_pages * page_size) // 2
    pending = [(i, rng.randint(1, max(1, biggest)), rng.randint(0, 16),
                rng.choice([None, None, 7])) for i in range(rng.randint(4, 12))]
    reqs = {}
    steps = 0
    while pending or sched.has_work():
        # requests arrive over time
        while pending and (rng.random() < 0.5 or not sched.has_work()):
            rid, plen, max_new, eos = pending.pop(0)
            reqs[rid] = Request(rid, [1] * plen, max_new, eos_token_id=eos)
            sched.add(reqs[rid])
            psched.add(rid, plen, max_new, eos)
        assert sched.has_work() == psched.has_work()
        if not sched.has_work():
            continue
        try:
            want = psched.schedule()
        except PlainOutOfPages:
            with pytest.raises(OutOfPages):
                sched.schedule()
            seen["refused"] = 1
            return seen                             # both refuse: a request that cannot fit
        plan = sched.schedule()
        assert [(e.request.id, e.start, e.count, e.samples) for e in plan] == want
        assert sched.preemption_count == psched.preemptions
        assert [r.id for r in sched.waiting] == psched.waiting
        assert sorted(r.id for r in sched.running) == sorted(psched.running)
        for e in plan:
            cache.reserve(e.request.id, e.count)
            pcache.reserve(e.request.id, e.count)
        for e in plan:
            cache.commit(e.request.id, e.count)
            pcache.commit(e.request.id, e.count)
        for rid in psched.running:
            assert cache.slot_of(rid) == pcache.req[rid]["slot"]
            assert cache.num_tokens(rid) == pcache.req[rid]["tokens"]
            for g in range(len(windows)):
                assert cache.table(rid, g) == pcache.req[rid]["tables"][g]
                seen["freed"] += pcache.req[rid]["tables"][g].count(FREED)
        sampled = {e.request.id: rng.choice([7, 11, 12, 13]) for e in plan if e.samples}
        done = sched.update(plan, sampled)
        assert [r.id for r in done] == psched.update(want, sampled)
        for r in done:
            assert r.finish_reason == psched.info[r.id]["done"]
            seen["eos"] += r.finish_reason == "eos"
        for g in range(len(windows)):
            assert cache.groups[g].pool.free_count == len(pcache.free[g])
        assert cache.slots.free_count == len(pcache.free_slots)
        cache.check()
        steps += 1
        assert steps < 5000
    assert all(r.phase == FINISHED for r in reqs.values())
    assert all(g.pool.free_count == g.pool.size for g in cache.groups)
    seen["preemptions"] = psched.preemptions
    seen["steps"] = steps
    return seen


@pytest.mark.parametrize("seed", SEEDS)
def test_host_library_against_the_plain_scheduler(seed):
    """Random workloads, pools so small that requests are preempted, windows that
    give pages back: the host library's plans, block tables and free counts equal
    those of the plain statement of the policy, step by step."""
    run_differential(seed)


def test_the_random_workloads_reach_the_hard_cases():
    total = {}
    for seed in SEEDS:
        for k, v in run_differential(seed).items():
            total[k] = total.get(k, 0) + v
    assert total["preemptions"] >= 10 and total["refused"] >= 1
    assert total["freed"] >= 10 and total["eos"] >= 3 and total["steps"] >= 300


def test_abort_gives_everything_back():
    """A request taken out while it waits, while it runs, and after it has finished:
    pages, slot and name go back, the others carry on."""
    cache, sched = make(num_pages=8, page_size=4, num_slots=2, max_num_seqs=2)
    a, b, c = (Request(n, list(range(6)), 3) for n in "abc")
    for r in (a, b, c):
        sched.add(r)
    plan = sched.schedule()                          # a and b run, c waits (two slots)
    assert [e.request.id for e in plan] == ["a", "b"]
    for e in plan:
        cache.reserve(e.request.id, e.count)
        cache.commit(e.request.id, e.count)
    sched.update(plan, {"a": 7, "b": 8})
    sched.abort(a)                                   # running
    sched.abort(c)                                   # waiting
    assert a.phase == FINISHED and a.finish_reason == "aborted" and c.finish_reason == "aborted"
    assert "a" not in cache.requests and len(cache.handles) == 1
    cache.check()
    drive(cache, sched)
    assert b.phase == FINISHED and b.finish_reason == "length" and len(b.output) == 3
    sched.abort(b)                                   # finished already: nothing happens
    assert b.finish_reason == "length"
    assert not sched.has_work() and len(cache.handles) == 0
    assert all(g.pool.free_count == g.pool.size for g in cache.groups)
    assert cache.slots.free_count == 2
