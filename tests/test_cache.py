"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of requests;
windows give pages back; state slots; the step bookkeeping around it."""
import random

import pytest
import torch

from jllm_serve_amd.cache import CacheEntryPlan, CacheManager, KvSpec, OutOfPages, PagePool, StateSpec
from fakes import FakeRunner
from jllm_serve_amd.engine.step import StepEntry, StepError


def manager(plans=None, page=4, tokens=64, reqs=4):
    plans = plans or [CacheEntryPlan(kv=KvSpec(2, 8, 0)), CacheEntryPlan(kv=KvSpec(2, 8, 0))]
    return CacheManager(plans, page, tokens, reqs, allocate=False)


def test_pool_basics():
    p = PagePool(3, 16)
    a, b, c = p.alloc(), p.alloc(), p.alloc()
    assert sorted([a, b, c]) == [0, 1, 2] and p.free_pages == 0
    with pytest.raises(OutOfPages, match="all 3 pages of 16 positions"):
        p.alloc()
    p.release(b)
    assert p.alloc() == b, "a freed page is usable at once"
    with pytest.raises(ValueError):
        p.release(7)
    p.release(a)
    with pytest.raises(ValueError, match="not held"):
        p.release(a)  # freed twice
    p.retain(c)
    p.release(c)
    assert p.refs(c) == 1 and p.free_pages == 1
    p.check()


def test_groups_follow_specs():
    plans = [CacheEntryPlan(kv=KvSpec(2, 8, 0)), CacheEntryPlan(kv=KvSpec(2, 8, 16)), CacheEntryPlan(kv=KvSpec(2, 8, 0)),
             CacheEntryPlan(cache_from=1), CacheEntryPlan(kv=None, state=StateSpec((3,), torch.float32))]
    m = CacheManager(plans, 4, 64, 2, dtype=torch.float32, device="cpu")
    assert [(g.spec.window, g.runs) for g in m.groups] == [(0, [0, 2]), (16, [1])]
    assert m.slots[3].group == 1 and not m.slots[3].writes and m.slots[1].writes
    assert m.slots[3].k_cache.data_ptr() == m.slots[1].k_cache.data_ptr(), "a run that reads another's cache gets its pages"
    assert m.slots[4].group is None and m.slots[4].state.shape == (2, 3)
    assert m.slots[0].k_cache.shape == (16, 2, 4, 8)
    with pytest.raises(ValueError):
        CacheManager([CacheEntryPlan(cache_from=0)], 4, 64, 2, allocate=False)
    with pytest.raises(ValueError, match="power of two"):
        CacheManager(plans, 12, 64, 2, allocate=False)


def test_begin_write_commit_close():
    m = manager()
    m.open("a")
    assert m.begin_write("a", 5) == 0 and len(m.table("a", 0)) == 2  # ceil(5/4) entries (KvSequence.java:116-146)
    m.commit("a", 5)
    assert m.begin_write("a", 3) == 5 and len(m.table("a", 0)) == 2
    m.commit("a", 3)
    m.begin_write("a", 1)
    assert len(m.table("a", 0)) == 3
    assert m.slot_indices("a", 0, 7, 2) == [m.table("a", 0)[1] * 4 + 3, m.table("a", 0)[2] * 4 + 0]
    m.rollback_write("a")
    assert len(m.table("a", 0)) == 2
    m.check()
    m.close("a")
    assert m.free_pages() == [16] and not m.has("a")
    with pytest.raises(KeyError):
        m.close("a")  # closed twice


def test_out_of_pages_is_atomic_across_groups():
    plans = [CacheEntryPlan(kv=KvSpec(1, 4, 0)), CacheEntryPlan(kv=KvSpec(1, 8, 0))]
    m = CacheManager(plans, 4, 16, 4, allocate=False)  # two groups of 4 pages
    m.open("a"); m.begin_write("a", 12); m.commit("a", 12)
    m.open("b")
    m.groups[1].pool.alloc()  # someone else holds the last page of group 1
    with pytest.raises(OutOfPages):
        m.begin_write("b", 4)
    assert m.table("b", 0) == [] and m.table("b", 1) == [] and m.free_pages() == [1, 0]
    m.check_groups = None


def test_window_gives_pages_back_and_reuses_them():
    plans = [CacheEntryPlan(kv=KvSpec(1, 4, 0)), CacheEntryPlan(kv=KvSpec(1, 4, 6))]
    m = CacheManager(plans, 4, 64, 2, allocate=False)
    m.open("a")
    for n in (5, 3, 1, 1, 9, 1):
        m.begin_write("a", n)
        m.commit("a", n)
        length = m.length("a")
        first = max(0, length + 1 - 6)  # the next query sees keys from here (Attention.java:68-71)
        t = m.table("a", 1)
        for b, page in enumerate(t):
            if (b + 1) * 4 <= first:
                assert page == -1, f"page of positions {b*4}..{b*4+3} is older than the window at length {length}"
            else:
                assert page >= 0
        assert all(p >= 0 for p in m.table("a", 0)), "the group without a window keeps everything"
        m.check()
    assert m.length("a") == 20 and m.groups[1].pool.used_pages == 2 and m.groups[0].pool.used_pages == 5
    assert m.pages_given_back_by_window == 3
    m.close("a")
    assert m.free_pages() == [16, 16]


def test_truncate():
    m = manager()
    m.open("a"); m.begin_write("a", 10); m.commit("a", 10)
    m.truncate("a", 5)
    assert m.length("a") == 5 and len(m.table("a", 0)) == 2 and m.free_pages() == [14]
    with pytest.raises(ValueError):
        m.truncate("a", 6)
    m.check()


def test_state_slots():
    m = CacheManager([CacheEntryPlan(state=StateSpec((2,), torch.float32))], 4, 16, 2, device="cpu")
    a = m.open("a"); b = m.open("b")
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(OutOfPages, match="request slots"):
        m.open("c")
    m.slots[0].state[a.state_slot] += 5
    m.close("a")
    c = m.open("c")
    assert c.state_slot == a.state_slot and float(m.slots[0].state[c.state_slot].abs().sum()) == 0, "a reused slot starts at zero"
    m.check()


def test_random_orders_keep_the_invariants():
    rng = random.Random(11)
    for trial in range(30):
        plans = [CacheEntryPlan(kv=KvSpec(1, 4, 0)), CacheEntryPlan(kv=KvSpec(1, 4, rng.choice([0, 5, 12])))]
        page = rng.choice([1, 2, 4, 8])
        m = CacheManager(plans, page, rng.choice([16, 40, 64]), rng.choice([2, 3, 5]), allocate=False)
        for g in m.groups:
            g.pool.shuffle_free(rng)
        live = []
        for op in range(200):
            r = rng.random()
            if r < 0.2 and len(live) < m.max_requests:
                rid = f"r{trial}.{op}"
                m.open(rid)
                live.append(rid)
            elif r < 0.8 and live:
                rid = rng.choice(live)
                n = rng.randrange(1, 12)
                before = [list(m.table(rid, gi)) for gi in range(len(m.groups))]
                try:
                    m.begin_write(rid, n)
                    if rng.random() < 0.15:
                        m.rollback_write(rid)
                    else:
                        m.commit(rid, n)
                except OutOfPages:
                    assert [list(m.table(rid, gi)) for gi in range(len(m.groups))] == before
            elif live:
                rid = live.pop(rng.randrange(len(live)))
                m.close(rid)
            m.check()
        for rid in live:
            m.close(rid)
        m.check()
        assert m.free_pages() == [g.pool.num_pages for g in m.groups], "every page came back"


def test_step_bookkeeping_and_errors():
    r = FakeRunner(pool_tokens=16, page_size=4, max_requests=2)
    out = r.step([StepEntry("a", [1, 2, 3], [2]), StepEntry("b", [4], [0])])
    assert out.shape == (2, 97) and r.cache.length("a") == 3 and r.cache.length("b") == 1
    with pytest.raises(StepError, match="twice"):
        r.step([StepEntry("a", [1]), StepEntry("a", [2])])
    with pytest.raises(StepError, match="outside the vocabulary"):
        r.step([StepEntry("a", [97])])
    with pytest.raises(StepError, match="wanted place"):
        r.step([StepEntry("a", [1], [1])])
    with pytest.raises(StepError, match="no tokens"):
        r.step([StepEntry("a", [])])
    # out of pages: nothing changes, not even for the entries before the one that failed
    with pytest.raises(OutOfPages):
        r.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(1, 14)))])
    assert r.cache.length("a") == 3 and r.cache.length("b") == 1 and len(r.cache.table("a", 0)) == 1
    r.cache.check()
    with pytest.raises(OutOfPages):
        r.step([StepEntry("c", [1])])  # a third request: no state slot
    assert not r.cache.has("c")
    r.finish("a"); r.finish("b"); r.finish("nobody")
    assert r.cache.free_pages() == [4]
