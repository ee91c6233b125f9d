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
    assert m.slots[3].rows["k"].data_ptr() == m.slots[1].rows["k"].data_ptr(), "a run that reads another's cache gets its pages"
    assert m.slots[4].group is None and m.slots[4].state.shape == (2 + 1, 3)  # the last row: padding rows of a captured step
    assert m.slots[0].rows["k"].shape == (16, 2, 4, 8) and m.slots[0].rows["v"].shape == (16, 2, 4, 8)
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


# ------------------------------------------------------------------------------------------ prefix sharing

def sharing_manager(page=16, tokens=4800, reqs=4, groups=1):
    plans = [CacheEntryPlan(kv=KvSpec(2, 8, 0)), CacheEntryPlan(kv=KvSpec(2, 8, 0))]
    if groups == 2:
        plans.append(CacheEntryPlan(kv=KvSpec(1, 16, 0)))
    m = CacheManager(plans, page, tokens, reqs, allocate=False, prefix_share=True)
    m.copied = []
    m.copy_page = lambda gi, src, dst, rows: m.copied.append((gi, src, dst, rows))
    return m


def compute(m, rid, tokens, n=None):
    """What a request does to the cache when it runs tokens[held : n): open, make room, commit, publish."""
    if not m.has(rid):
        m.open(rid)
    n = len(tokens) if n is None else n
    held = m.length(rid)
    m.begin_write(rid, n - held)
    m.commit(rid, n - held)
    m.publish(rid, tokens[:n])


def test_prefix_vectors_of_the_reference():
    """150 positions in blocks of 16: nine published blocks, a second sequence finds and adopts 144
    (T/cpu/PagedKvTest.java:209-225). 46 positions: match over 45 finds the two full blocks, 32; a prompt that
    differs from token 21 on shares 21, the 5 rows of the second block by a copy (T/PagedKvChecks.java:188-209)."""
    rng = random.Random(5)
    tokens = [rng.randrange(500) for _ in range(300)]
    m = sharing_manager()
    compute(m, "s1", tokens, 150)
    assert m.published_pages("s1") == 9
    found = m.match(tokens, 150)
    assert (found.tokens, found.nodes, found.idle_nodes, found.partial) == (144, 9, 0, 0)
    m.open("s2")
    assert m.adopt("s2", tokens, found.tokens) == 144 and m.length("s2") == 144
    assert m.table("s2", 0) == m.table("s1", 0)[:9], "the same nine pages, not copies"
    m.check()
    assert m.groups[0].pool.used_pages == 10, "two sequences of 150 positions hold ten pages"
    compute(m, "s2", tokens[:144] + [7] * 7, 151)  # s2 writes its own tail from 144 on
    assert m.table("s2", 0)[9] != m.table("s1", 0)[9]
    m.check()

    m = sharing_manager()
    compute(m, "a", tokens, 20)
    compute(m, "a", tokens, 46)
    assert m.match(tokens, 45).tokens == 32
    m.open("b")
    assert m.adopt("b", tokens, 32) == 32
    other = tokens[:21] + [(t + 101) % 500 for t in tokens[21:]]
    fork = m.match(other, 40)
    assert (fork.tokens, fork.nodes, fork.partial) == (21, 1, 5)
    m.open("c")
    assert m.adopt("c", other, fork.tokens) == 21
    src, dst = m.table("a", 0)[1], m.table("c", 0)[1]
    assert src != dst and m.copied == [(0, src, dst, 5)], "a fork inside a block copies the rows it shares"
    m.check()
    # a rewinds into block 1 and goes on differently: it gets a page of its own, b and c keep theirs
    before = (list(m.table("b", 0)), list(m.table("c", 0)))
    m.truncate("a", 25)
    m.begin_write("a", 6)
    assert m.copied[-1] == (0, src, m.table("a", 0)[1], 9) and m.table("a", 0)[1] != src
    m.commit("a", 6)
    assert (m.table("b", 0), m.table("c", 0)) == before and m.table("b", 0)[1] == src
    m.check()
    assert m.groups[0].pool.used_pages < 3 * 3, "three sequences of about 46 positions share pages"


def test_prefix_pages_stay_as_cache_and_are_evicted_oldest_leaf_first():
    m = sharing_manager(page=4, tokens=40, reqs=4)  # ten pages
    x = list(range(100, 116))  # four pages
    y = list(range(200, 212))  # three pages
    compute(m, "x", x + [1])
    compute(m, "y", y + [2])
    m.close("x")
    m.close("y")
    m.check()
    assert m.groups[0].pool.used_pages == 7 and m.tree.idle == 7
    assert m.free_pages() == [10], "pages that only the tree holds can be had"
    assert m.match(x, len(x)).idle_nodes == 4  # also makes x the more recently used chain
    x_pages = [n.pages[0] for n in m.tree.walk() if n.tokens[0] < 200]
    m.open("z")
    m.begin_write("z", 16)  # four pages: three free ones, then the deepest page of y (used longest ago)
    assert m.tree.evictions == 1 and m.tree.idle == 6
    assert m.match(y, len(y)).tokens == 8 and m.match(x, len(x)).tokens == 16
    m.commit("z", 16)
    m.begin_write("z", 40 - 16)  # the whole pool: everything cached goes, leaves before their parents
    assert m.tree.nodes == 0 and m.tree.evictions == 7 and m.free_pages() == [0]
    assert set(x_pages) <= set(m.table("z", 0))
    m.check()
    with pytest.raises(OutOfPages):
        m.open("w")
        m.begin_write("w", 1)
    m.close("w")
    m.close("z")
    m.check()
    assert m.groups[0].pool.used_pages == 0


def test_used_pages_are_never_evicted_and_adoption_protects_its_source():
    m = sharing_manager(page=4, tokens=24, reqs=3)  # six pages
    x = list(range(50, 62))
    compute(m, "x", x + [1])  # 4 pages held, 3 published
    m.open("y")
    with pytest.raises(OutOfPages):
        m.begin_write("y", 12)  # needs 3, two are free and x's are in use
    m.check()
    assert m.tree.nodes == 3 and m.table("y", 0) == []
    assert m.adopt("y", x[:6] + [0, 0], 6) == 6, "one shared page and a copy of two rows"
    assert m.table("y", 0)[0] == m.table("x", 0)[0] and m.copied[-1][3] == 2
    m.check()
    m.close("x")
    assert m.tree.idle == 2, "the page y goes through stays in use"
    m.open("v")
    m.begin_write("v", 16)  # one free page, x's own tail page and the two idle pages; y's stay
    assert m.tree.nodes == 1 and m.free_pages() == [0]
    m.check()


def test_publishing_the_same_tokens_twice_keeps_one_copy():
    m = sharing_manager(page=4, tokens=64, reqs=3, groups=2)
    t = list(range(30, 43))
    m.open("a"); m.begin_write("a", 13); m.commit("a", 13)
    m.open("b"); m.begin_write("b", 13); m.commit("b", 13)
    m.publish("a", t)
    own = list(m.table("b", 1))
    m.publish("b", t)
    assert m.tree.dedups == 3 and m.table("b", 0)[:3] == m.table("a", 0)[:3] and m.table("b", 1)[:3] == m.table("a", 1)[:3]
    assert m.table("b", 1)[3] == own[3] and all(m.groups[1].pool.refs(p) == 0 for p in own[:3])
    m.check()
    assert [g.pool.used_pages for g in m.groups] == [5, 5]
    m.close("a"); m.close("b")
    m.check()
    assert m.drop_cached() == 3 and [g.pool.used_pages for g in m.groups] == [0, 0]


def test_models_that_cannot_share_run_without():
    windowed = CacheManager([CacheEntryPlan(kv=KvSpec(2, 8, 16))], 4, 64, 2, allocate=False, prefix_share=True)
    assert not windowed.sharing and "window" in windowed.sharing_refused
    stateful = CacheManager([CacheEntryPlan(kv=KvSpec(2, 8, 0)), CacheEntryPlan(state=StateSpec((3,)))], 4, 64, 2,
                            allocate=False, prefix_share=True)
    assert not stateful.sharing and "state" in stateful.sharing_refused
    assert windowed.match([1, 2, 3, 4, 5]).tokens == 0
    plain = manager()
    assert not plain.sharing and plain.sharing_refused == ""


def test_random_orders_with_sharing_keep_the_invariants():
    rng = random.Random(11)
    for trial in range(20):
        B = rng.choice([2, 4, 8])
        m = sharing_manager(page=B, tokens=B * rng.choice([12, 20, 40]), reqs=4, groups=rng.choice([1, 2]))
        stems = [[rng.randrange(50) for _ in range(rng.randrange(3, 40))] for _ in range(3)]
        live = {}
        for op in range(300):
            kind = rng.random()
            if kind < 0.3 and len(live) < 4:
                rid = f"r{trial}-{op}"
                tokens = list(rng.choice(stems))[:rng.randrange(2, 40)] + [rng.randrange(50) for _ in range(rng.randrange(0, 12))]
                m.open(rid)
                found = m.match(tokens, len(tokens) - 1)
                got = m.adopt(rid, tokens, found.tokens)
                assert got <= found.tokens and got == m.length(rid)
                live[rid] = tokens
            elif kind < 0.75 and live:
                rid = rng.choice(list(live))
                tokens = live[rid]
                n = min(len(tokens) - m.length(rid), rng.randrange(1, 9))
                if n <= 0:
                    tokens.append(rng.randrange(50))
                    n = 1
                try:
                    m.begin_write(rid, n)
                except OutOfPages:
                    m.check()
                    m.close(rid)
                    del live[rid]
                    continue
                m.commit(rid, n)
                m.publish(rid, tokens[:m.length(rid)])
            elif kind < 0.85 and live:
                rid = rng.choice(list(live))
                keep = rng.randrange(0, m.length(rid) + 1)
                m.truncate(rid, keep)
                live[rid] = live[rid][:keep] + [rng.randrange(50) for _ in range(rng.randrange(1, 6))]
            elif live:
                rid = rng.choice(list(live))
                m.close(rid)
                del live[rid]
            m.check()
            assert all(f == g.pool.free_pages + m.tree.idle for f, g in zip(m.free_pages(), m.groups))
        for rid in list(live):
            m.close(rid)
        m.check()
        assert all(g.pool.used_pages == m.tree.nodes for g in m.groups), "what is left is what the tree holds"
        m.drop_cached()
        assert all(g.pool.used_pages == 0 for g in m.groups) and m.tree.nodes == 0
        m.check()


def test_pool_vectors_of_the_reference():
    """The numbers of the reference's pool tests (T/KvPoolTest.java:156-170, :202-231, :255-302) with pages of 16:
    4,100 tokens take 257 pages and a second conversation with the same 4,000-token start finds it; a fork at 40
    shares 40 tokens, the 8 of the third page by a copy; a finished conversation of 160 tokens stays as 10 cached
    pages and is found; four conversations of 13 pages do not fit a pool of 40 and the pool says so; afterwards
    nothing is held."""
    rng = random.Random(1)
    sysp = [rng.randrange(1000) for _ in range(4000)]
    m = sharing_manager(page=16, tokens=16 * 1000, reqs=4)
    ta = sysp + [rng.randrange(1000) for _ in range(100)]
    compute(m, "a", ta)
    assert m.groups[0].pool.used_pages == (4100 + 15) // 16 == 257
    tb = sysp + [rng.randrange(1000) for _ in range(100)]
    assert m.match(tb, len(tb) - 1).tokens >= 4000

    m = sharing_manager(page=16, tokens=16 * 200, reqs=4)
    t = [rng.randrange(1000) for _ in range(200)]
    compute(m, "a", t)
    t2 = t[:40] + [1000 + i for i in range(100)]
    found = m.match(t2, len(t2) - 1)
    assert found.tokens == 40 and found.partial == 8
    m.open("b")
    assert m.adopt("b", t2, found.tokens) == 40 and m.copied[-1][3] == 8, "adopting copies the 8 shared rows"
    compute(m, "b", t2)
    m.open("c")
    assert m.adopt("c", t, m.match(t, 199).tokens) >= 192
    table_c = list(m.table("c", 0))
    m.truncate("a", 70)  # a rewinds to 70 and continues differently: c keeps what it adopted
    m.begin_write("a", 30)
    m.commit("a", 30)
    assert m.table("c", 0) == table_c and m.table("a", 0)[4] != table_c[4] and m.copied[-1][3] == 70 % 16
    used = m.groups[0].pool.used_pages
    m.truncate("a", 16)
    assert m.groups[0].pool.used_pages < used, "truncate releases pages"
    m.check()

    m = sharing_manager(page=16, tokens=16 * 40, reqs=4)
    s160 = [rng.randrange(1000) for _ in range(160)]
    compute(m, "a", s160)
    m.close("a")
    st = m.stats()
    assert st["prefix"]["idle"] == 10 and st["groups"][0]["used"] == 10 and m.free_pages() == [40], "a finished conversation stays cached"
    assert m.match(s160, 159).tokens >= 144
    with pytest.raises(OutOfPages, match="all 40 pages"):
        for i in range(4):  # 13 pages each: 52 > 40
            m.open(f"h{i}")
            m.begin_write(f"h{i}", 200)
            m.commit(f"h{i}", 200)
    assert m.tree.evictions == 10, "the cached pages went first"
    for rid in list(m.requests):
        m.close(rid)
    m.check()
    assert m.groups[0].pool.used_pages == 0, "everything is released afterwards"
