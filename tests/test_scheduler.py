"""The scheduler's decisions, with no model: a loop that pretends every step runs
(in the style of the reference's scheduler tests, crates/denno-server/tests/scheduler.rs:33-61)."""
import pytest

from denno_beta_amd.cache import PAGED, CacheManager, GroupLayout
from denno_beta_amd.engine.scheduler import Scheduler, SchedulerError


def mk(n_pages=64, page=16, max_live=4, budget=64, chunk=32, policy="preempt", positions=256, window=0):
    cache = CacheManager([GroupLayout(PAGED, n_pages, page, window)], max_live)
    return cache, Scheduler(cache, max_live=max_live, max_batch_tokens=budget, prefill_chunk=chunk,
                            policy=policy, max_positions=positions)


def run(cache, s, max_steps=10000, on_step=None):
    """Steps until nothing is left; -> (list of plans, {rid: tokens generated}, preemptions)."""
    plans, generated, pre = [], {}, []
    for _ in range(max_steps):
        if s.n_waiting() + s.n_running() == 0:
            return plans, generated, pre
        plan, p = s.schedule()
        pre += p
        assert plan, "nothing can run"
        plans.append(plan)
        for e in plan:
            assert e.start == s.computed(e.rid) and e.start + e.count <= s.known(e.rid)
            assert cache.block_table(e.rid, 0).size * 16 >= e.start + e.count or True
            s.step_done(e.rid, e.count)
        for e in plan:
            if e.samples:
                generated[e.rid] = generated.get(e.rid, 0) + 1
                if s.token_sampled(e.rid):
                    s.finish(e.rid)
        cache.check()
        if on_step:
            on_step(plan)
    raise AssertionError("did not finish")


def test_admission_errors_and_clamp():
    _, s = mk(positions=100)
    with pytest.raises(SchedulerError, match="empty"):
        s.add(0, 0, 5)
    with pytest.raises(SchedulerError, match="longer"):
        s.add(0, 101, 5)
    # max_new is clamped to the positions left (crates/denno-engine/src/engine.rs:865-881)
    assert s.add(0, 90, 50) == 10 and s.add(1, 100, 5) == 0 and s.add(2, 10, 5) == 5
    with pytest.raises(SchedulerError, match="in use"):
        s.add(2, 10, 5)
    _, small = mk(n_pages=2)
    with pytest.raises(SchedulerError, match="even alone"):
        small.add(0, 40, 1)
    assert small.add(1, 30, 3) == 3            # 30 + 2 fed tokens fit two pages


def test_one_prompt_in_portions_then_decodes():
    cache, s = mk(chunk=32, budget=64)
    s.add(0, 70, 3)
    plans, gen, _ = run(cache, s)
    assert [(e.start, e.count, e.samples) for p in plans for e in p] == [
        (0, 32, False), (32, 32, False), (64, 6, True), (70, 1, True), (71, 1, True)]
    assert gen == {0: 3} and cache.live() == 0 and cache.free_pages(0) == 64


def test_decodes_first_then_portions_under_the_budget():
    cache, s = mk(chunk=32, budget=40, max_live=4)
    s.add(0, 5, 50)
    s.add(1, 100, 2)
    first, _ = s.schedule()
    # first come first served: request 0 whole, then request 1 with what is left of the budget
    assert [(e.rid, e.count) for e in first] == [(0, 5), (1, 32)]
    for e in first:
        s.step_done(e.rid, e.count)
    s.token_sampled(0)
    second, _ = s.schedule()
    assert [(e.rid, e.start, e.count, e.samples) for e in second] == [(0, 5, 1, True), (1, 32, 32, False)]
    assert sum(e.count for e in second) <= 40


def test_live_cap_and_fifo():
    cache, s = mk(max_live=2, budget=256, chunk=64)
    for rid in range(5):
        s.add(rid, 10, 2 + rid)
    order = []
    plans, gen, _ = run(cache, s, on_step=lambda plan: order.extend(e.rid for e in plan if e.start == 0))
    assert order == [0, 1, 2, 3, 4]
    assert all(len(p) <= 2 for p in plans)
    assert gen == {r: 2 + r for r in range(5)}      # uneven completion (crates/denno-engine/src/engine.rs:2503-2542)


def test_reserve_policy_never_runs_out():
    cache, s = mk(n_pages=8, policy="reserve", max_live=4, budget=256, chunk=64)
    for rid in range(4):
        s.add(rid, 30, 35)          # peak 64 tokens = 4 pages each: two fit at a time
    seen = []
    plans, gen, pre = run(cache, s, on_step=lambda plan: seen.append(len(plan)))
    assert pre == [] and max(seen) == 2 and gen == {r: 35 for r in range(4)}
    assert cache.free_pages(0) == 8


def test_preempt_policy_recomputes_the_youngest():
    cache, s = mk(n_pages=8, policy="preempt", max_live=4, budget=256, chunk=64)
    for rid in range(3):
        s.add(rid, 30, 40)          # 69 tokens = 5 pages each at the end; the pool has 8
    plans, gen, pre = run(cache, s)
    assert gen == {r: 40 for r in range(3)}
    assert pre and 0 not in pre                     # the oldest is never preempted
    # a preempted request starts again from position 0 with all its known tokens
    restarts = [e for p in plans for e in p if e.start == 0]
    assert len(restarts) == 3 + len(pre)
    assert cache.free_pages(0) == 8 and cache.live() == 0


def test_prefill_only_request():
    cache, s = mk()
    s.add(0, 20, 0)
    plan, _ = s.schedule()
    assert [(e.count, e.samples) for e in plan] == [(20, True)]
    s.step_done(0, 20)
    with pytest.raises(SchedulerError):
        s.token_sampled(0)          # nothing may be sampled: max_new is 0
    s.finish(0)
    assert cache.live() == 0


def test_finish_of_a_waiting_request_and_unknown():
    cache, s = mk(max_live=1)
    s.add(0, 10, 5), s.add(1, 10, 5)
    s.schedule()
    assert s.n_running() == 1 and s.n_waiting() == 1
    s.finish(1)
    assert s.n_waiting() == 0
    with pytest.raises(SchedulerError, match="unknown"):
        s.finish(1)
    assert s.known(1) == -1 and s.known(0) == 10      # asking is no error
    s.finish(0)
    assert cache.live() == 0 and cache.free_pages(0) == 64


def test_windowed_pool_lets_long_requests_share_few_pages():
    cache, s = mk(n_pages=6, page=16, window=32, budget=64, chunk=16, positions=1024, max_live=2)
    s.add(0, 200, 50)
    s.add(1, 150, 30)
    plans, gen, pre = run(cache, s)
    assert gen == {0: 50, 1: 30} and pre == []
