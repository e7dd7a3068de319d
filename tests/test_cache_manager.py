"""The cache manager: no page lost, held twice or freed twice, under any order of requests.
Unit vectors after the reference's cache tests (crates/denno-engine/src/kv_cache.rs:371-468),
turned from rows of one buffer into pages of a pool."""
import random

import numpy as np

import pytest

from denno_beta_amd.cache import PAGED, STATE, CacheError, CacheManager, GroupLayout, OutOfPages


def mk(n_pages=8, page=16, window=0, max_requests=4, extra=()):
    return CacheManager([GroupLayout(PAGED, n_pages, page, window), *extra], max_requests)


def test_new_cache_is_empty():
    m = mk()
    assert m.free_pages(0) == 8 and m.live() == 0
    m.check()


def test_add_reserve_commit_release():
    m = mk()
    slot = m.add(7)
    assert slot == 0 and m.length(7) == 0 and m.block_table(7, 0).tolist() == []
    m.reserve(7, 17)
    assert m.block_table(7, 0).tolist() == [0, 1] and m.free_pages(0) == 6
    m.commit(7, 17)
    assert m.length(7) == 17
    m.reserve(7, 32)            # still inside the second page
    assert m.free_pages(0) == 6
    m.reserve(7, 33)
    assert m.block_table(7, 0).tolist() == [0, 1, 2]
    assert m.release(7) and m.free_pages(0) == 8 and m.live() == 0
    m.check()


def test_commit_needs_pages_and_cannot_shrink():
    m = mk()
    m.add(1)
    with pytest.raises(CacheError):
        m.commit(1, 5)          # nothing reserved
    m.reserve(1, 20)
    m.commit(1, 20)
    with pytest.raises(CacheError):
        m.commit(1, 10)
    with pytest.raises(CacheError):
        m.reserve(1, 10)


def test_out_of_pages_changes_nothing():
    m = mk(n_pages=4)
    m.add(1), m.add(2)
    m.reserve(1, 48)
    with pytest.raises(OutOfPages):
        m.reserve(2, 40)        # wants 3, one is free
    assert m.free_pages(0) == 1 and m.block_table(2, 0).tolist() == []
    assert not m.try_reserve(2, 17) and m.try_reserve(2, 16)
    assert m.free_pages(0) == 0
    m.check()


def test_stale_and_double_release_are_no_ops():
    # crates/denno-engine/src/engine.rs:3445-3479
    m = mk()
    m.add(1)
    m.reserve(1, 30)
    assert m.release(1) is True
    assert m.release(1) is False and m.release(99) is False
    assert m.free_pages(0) == 8
    m.check()


def test_slots_and_generations():
    m = mk(max_requests=2)
    a, b = m.add(10), m.add(11)
    assert {a, b} == {0, 1}
    with pytest.raises(CacheError, match="slot"):
        m.add(12)
    with pytest.raises(CacheError, match="live already"):
        m.add(10)
    g = m.generation(a)
    m.release(10)
    assert m.add(12) == a and m.generation(a) == g + 1      # the slot is used again, under a new generation


def test_a_slot_record_starts_at_zero_for_the_next_request():
    m = mk(max_requests=1)
    slot = m.add(10)
    m.reserve(10, 20), m.commit(10, 20)
    m.set_rng(10, 2 ** 63 + 5, 3)
    m.note_sampled(10, 77)
    st = m.state(10)
    assert (st.num_computed, st.last_token, st.rng_seed, st.rng_drawn) == (20, 77, 2 ** 63 + 5, 4)
    seeds, drawn = m.rng_states(np.asarray([10], dtype=np.int64))
    assert seeds.tolist() == [2 ** 63 + 5] and drawn.tolist() == [4]
    m.release(10)
    with pytest.raises(CacheError, match="no live request"):
        m.state(10)
    assert m.add(11) == slot
    st = m.state(11)
    assert (st.num_computed, st.last_token, st.rng_seed, st.rng_drawn) == (0, -1, 0, 0)


def test_freed_pages_are_used_again():
    m = mk(n_pages=4)
    m.add(1)
    m.reserve(1, 64)
    first = m.block_table(1, 0).tolist()
    assert m.reuse_count(0) == 0
    m.release(1)
    m.add(2)
    m.reserve(2, 64)
    assert sorted(m.block_table(2, 0).tolist()) == sorted(first) and m.reuse_count(0) == 4


def test_window_gives_pages_back_as_it_passes():
    m = mk(n_pages=8, page=4, window=6)
    m.add(1)
    m.reserve(1, 8)
    m.commit(1, 8)              # the next query (position 8) reads keys 3..8: block 0 still holds key 3
    assert m.block_table(1, 0).tolist() == [0, 1] and m.pages_held(1, 0) == 2
    m.reserve(1, 10)
    m.commit(1, 10)             # next query reads keys 5..: block 0 (keys 0-3) has passed
    assert m.block_table(1, 0).tolist() == [-1, 1, 2] and m.free_pages(0) == 6
    for n in range(11, 40):
        m.reserve(1, n)
        m.commit(1, n)
        assert m.pages_held(1, 0) <= 3
        m.check()
    assert m.block_table(1, 0).tolist()[:8] == [-1] * 8
    m.release(1)
    assert m.free_pages(0) == 8
    m.check()


def test_groups_have_pools_of_their_own():
    m = CacheManager([GroupLayout(PAGED, 8, 16, 0), GroupLayout(PAGED, 3, 16, 16), GroupLayout(STATE)], 2)
    m.add(1)
    m.reserve(1, 40)
    assert m.free_pages(0) == 5 and m.free_pages(1) == 0
    m.add(2)
    with pytest.raises(OutOfPages):
        m.reserve(2, 1)         # the windowed pool is empty, so nothing is taken from the other either
    assert m.free_pages(0) == 5
    m.commit(1, 40)             # window 16: keys 25.. are read; blocks 0 (0-15) has passed
    assert m.block_table(1, 1).tolist() == [-1, 1, 2] and m.block_table(1, 0).tolist() == [0, 1, 2]
    m.reserve(2, 1)
    m.check()
    assert m.pages_peak(0, 100, 32) == 7 and m.pages_peak(1, 100, 32) == 4 and m.pages_peak(2, 100, 32) == 0


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted(seed):
    rng = random.Random(seed)
    window = [0, 0, 24, 5, 0, 40][seed]
    m = CacheManager([GroupLayout(PAGED, 24, 8, 0), GroupLayout(PAGED, 12, 8, window)], 5)
    live, next_rid = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            m.add(next_rid)
            live[next_rid] = 0
            next_rid += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = live[rid] + rng.choice([1, 1, 1, 2, 7, 19])
            if m.try_reserve(rid, n):
                m.commit(rid, n)
                live[rid] = n
                tab = m.block_table(rid, 0).tolist()
                assert len(tab) == -(-n // 8) and all(p >= 0 for p in tab)
        elif op < 0.95 and live:
            rid = rng.choice(list(live))
            assert m.release(rid)
            del live[rid]
        else:
            assert m.release(next_rid + 1000) is False
        m.check()
        held = sum(m.pages_held(r, 0) for r in live)
        assert held + m.free_pages(0) == 24
        assert sum(m.pages_held(r, 1) for r in live) + m.free_pages(1) == 12
    for rid in list(live):
        m.release(rid)
    assert m.free_pages(0) == 24 and m.free_pages(1) == 12
    m.check()


def _arr(vals, dtype):
    import numpy as np
    return np.asarray(vals, dtype=dtype)


def test_a_whole_step_in_one_call_each_agrees_with_the_calls_per_request():
    """lengths, reserve_step, max_blocks, step_tables and commit_step against the same done request
    by request, over random steps of portions and single tokens, with a window in one group."""
    import numpy as np
    rng = random.Random(5)
    layouts = [GroupLayout(PAGED, 40, 16, 0), GroupLayout(STATE), GroupLayout(PAGED, 40, 8, 20)]
    a, b = CacheManager(layouts, 6), CacheManager(layouts, 6)
    live = []
    for step in range(200):
        if len(live) < 5 and rng.random() < 0.3:
            rid = 100 + step
            assert a.add(rid) == b.add(rid)
            live.append(rid)
        if live and rng.random() < 0.1:
            rid = live.pop(rng.randrange(len(live)))
            assert a.release(rid) and b.release(rid)
        chosen = [r for r in live if rng.random() < 0.7]
        rng.shuffle(chosen)
        chosen = [r for r in chosen if a.length(r) < 100]
        if not chosen:
            continue
        rids = _arr(chosen, np.int64)
        counts = _arr([rng.choice([1, 1, 2, 5, 17]) for _ in chosen], np.int32)
        starts = a.lengths(rids)
        assert starts.tolist() == [b.length(r) for r in chosen]
        slots = a.reserve_step(rids, starts + counts)
        for r, s, c in zip(chosen, starts.tolist(), counts.tolist()):
            b.reserve(r, s + c)
        assert slots.tolist() == [b.slot(r) for r in chosen]
        for g in (0, 2):
            ps = layouts[g].page_size
            tables = [b.block_table(r, g) for r in chosen]
            mb = a.max_blocks(g, rids)
            assert mb == max(len(t) for t in tables)
            rows = len(chosen) + 2                       # as a graph's bucket has rows beyond the requests
            bt = np.full((rows, mb), 99, dtype=np.int32)
            sm = np.full(int(counts.sum()) + 3, 99, dtype=np.int32)
            assert a.step_tables(g, rids, starts, counts, bt, sm) == -1
            want_bt = np.full((rows, mb), -1, dtype=np.int32)
            want_sm = []
            for i, (t, s, c) in enumerate(zip(tables, starts.tolist(), counts.tolist())):
                want_bt[i, :len(t)] = t
                want_sm += [int(t[p // ps]) * ps + p % ps for p in range(s, s + c)]
            assert (bt == want_bt).all()
            assert sm.tolist() == want_sm + [-1, -1, -1]
        a.commit_step(rids, starts + counts)
        for r, s, c in zip(chosen, starts.tolist(), counts.tolist()):
            b.commit(r, s + c)
        a.check(), b.check()
        assert [a.free_pages(g) for g in (0, 2)] == [b.free_pages(g) for g in (0, 2)]
    for r in live:
        a.release(r)
    a.check()
    assert a.free_pages(0) == 40 and a.free_pages(2) == 40


def test_a_step_that_runs_out_of_pages_names_the_request_and_keeps_the_earlier_ones():
    import numpy as np
    m = mk(n_pages=3)
    m.add(1), m.add(2), m.add(3)
    rids = _arr([1, 2, 3], np.int64)
    with pytest.raises(OutOfPages, match="request 2"):
        m.reserve_step(rids, _arr([16, 48, 16], np.int32))      # 1 + 3 pages of 3
    assert m.block_table(1, 0).tolist() == [0] and m.block_table(2, 0).tolist() == [] and m.free_pages(0) == 2
    with pytest.raises(CacheError, match="request 9"):
        m.lengths(_arr([1, 9], np.int64))
    m.check()


def test_step_tables_refuse_a_token_without_a_page():
    import numpy as np
    m = mk(n_pages=8, page=4, window=4)
    m.add(1)
    m.reserve(1, 12), m.commit(1, 12)        # the window has passed the first block
    assert m.block_table(1, 0).tolist()[0] == -1
    rids, one = _arr([1], np.int64), _arr([1], np.int32)
    bt, sm = np.zeros((1, 3), dtype=np.int32), np.zeros(1, dtype=np.int32)
    assert m.step_tables(0, rids, _arr([2], np.int32), one, bt, sm) == 0        # position 2: its page was given back
    assert m.step_tables(0, rids, _arr([12], np.int32), one, bt, sm) == 0       # position 12: never reserved
    assert m.step_tables(0, rids, _arr([11], np.int32), one, bt, sm) == -1 and sm[0] == bt[0, 2] * 4 + 3
    assert m.step_tables(0, rids, _arr([11], np.int32), one, np.zeros((1, 2), dtype=np.int32), sm) == 0   # table too small
