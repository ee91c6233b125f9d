"""The cache manager: paged keys and values per group of layers, block tables per request, state slots.

What is kept of the reference's design (docs/24-paged-kv-cache.md:53-72; kv/KvSequence.java:116-146): a
page holds ``page_size`` consecutive positions of every layer of its group; the address of position p is
page ``table[p // page_size]``, row ``p % page_size``; before a step writes positions [pos, pos + n) the
table is extended to ceil((pos + n) / page_size) entries.

What is different: the reference has one group and refuses models whose layers differ
(model/Decoder.java:40-49). Here every cache-owning run of the layer schedule declares a ``PageSpec``
(named per-position tensors and a window; ``KvSpec`` makes the one of attention); runs with equal specs form a group with its own pool, storage and block table per request. A group with
a window gives pages back as soon as every position in them is older than any later query can see
(model/Attention.java:68-71: the query at p sees keys from max(0, p + 1 - window)). Beside the pages
there are fixed-size state slots: one index per live request into per-run state tensors.

With ``prefix_share`` the full pages of a request are published in a prefix tree (cache/prefix.py) and a
later request whose tokens start the same way takes them over instead of computing them
(kv/KvPool.java:375-587). Pages that only the tree holds are cache: they count as free and are evicted,
oldest use first, when a page is needed. Sharing is off for a model with a window (pages that a window has
passed are gone) or with per-request state (a state cannot start in the middle: model/Backend.java:113-117).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .tables import BlockTable, TableArena
from .pages import OutOfPages, PagePool
from .prefix import PrefixMatch, PrefixNode, PrefixTree


@dataclass(frozen=True)
class CacheRow:
    """One tensor that a cache-owning layer run keeps for every position: ``shape`` is what one position holds;
    in a page the positions lie at ``position_axis`` among these axes, so the run's storage is
    ``[pages, *shape[:position_axis], page_size, *shape[position_axis:]]``. ``dtype`` None: the run's cache type."""

    name: str
    shape: Tuple[int, ...]
    position_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def __post_init__(self):
        if not self.shape or any(int(d) < 1 for d in self.shape) or not 0 <= self.position_axis <= len(self.shape):
            raise ValueError(f"cache row '{self.name}': shape {self.shape} with the positions at axis {self.position_axis}")

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        a = self.position_axis
        return tuple(self.shape[:a]) + (page_size,) + tuple(self.shape[a:])


@dataclass(frozen=True)
class PageSpec:
    """What one cache-owning layer run stores per position: any number of named tensors (attention: a key and a
    value; a mixer with one compressed row: one), and the window after which positions are never read again."""

    rows: Tuple[CacheRow, ...]
    window: int = 0  # 0 = all earlier positions stay visible

    def __post_init__(self):
        names = [r.name for r in self.rows]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a page spec needs rows with distinct names, got {names}")


def KvSpec(kv_heads: int, head_dim: int, window: int = 0) -> PageSpec:
    """The page spec of attention: a key and a value of [kv_heads, head_dim] per position, heads outermost in a page
    (``[pages, kv_heads, page_size, head_dim]``: the keys of one head lie together)."""
    return PageSpec((CacheRow("k", (kv_heads, head_dim), 1), CacheRow("v", (kv_heads, head_dim), 1)), window)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size that one layer run keeps (shape without the slot dimension)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class CacheEntryPlan:
    """One run of the layer schedule as the cache manager sees it."""

    kv: Optional[PageSpec] = None  # None: this run owns no pages
    cache_from: Optional[int] = None  # reads the pages of that earlier run
    state: Optional[StateSpec] = None


@dataclass
class LayerSlot:
    """What one run of the schedule is handed at every step."""

    group: Optional[int] = None
    rows: Dict[str, torch.Tensor] = field(default_factory=dict)  # row name -> [pages, *page shape] of this run
    page_size: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None  # [slots, *shape]


class KvGroup:
    def __init__(self, gid: int, spec: PageSpec, runs: List[int], num_pages: int, page_size: int):
        self.gid = gid
        self.spec = spec
        self.runs = runs
        self.pool = PagePool(num_pages, page_size)
        self.tables: Optional[TableArena] = None  # the requests' block tables, one row per request slot
        self.storage: Dict[str, torch.Tensor] = {}  # row name -> [len(runs), pages, *page shape]


@dataclass
class RequestCache:
    rid: object
    length: int = 0  # positions held
    state_slot: int = -1
    tables: List[BlockTable] = field(default_factory=list)  # per group: page ids, -1 = given back
    released: List[int] = field(default_factory=list)  # per group: leading table entries already given back
    path: List[PrefixNode] = field(default_factory=list)  # tree nodes that the leading table entries are


class CacheManager:
    def __init__(self, plans: Sequence[CacheEntryPlan], page_size: int, pool_tokens: int, max_requests: int,
                 dtype: torch.dtype = torch.float32, device="cpu", allocate: bool = True, prefix_share: bool = False):
        if page_size < 1 or (page_size & (page_size - 1)) != 0:
            raise ValueError(f"page size must be a power of two, got {page_size}")
        self.page_size = page_size
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = torch.device(device)
        self.num_pages = max(1, -(-pool_tokens // page_size))
        self.groups: List[KvGroup] = []
        self.slots: List[LayerSlot] = []
        by_spec: Dict[KvSpec, KvGroup] = {}
        owner_index: Dict[int, Tuple[int, int]] = {}  # run -> (group, index within group)
        for i, p in enumerate(plans):
            if p.cache_from is not None:
                if p.cache_from not in owner_index:
                    raise ValueError(f"layer run {i} reads the cache of run {p.cache_from}, which owns none")
                continue
            if p.kv is None:
                continue
            g = by_spec.get(p.kv)
            if g is None:
                g = KvGroup(len(self.groups), p.kv, [], self.num_pages, page_size)
                by_spec[p.kv] = g
                self.groups.append(g)
            owner_index[i] = (g.gid, len(g.runs))
            g.runs.append(i)
        if allocate:
            for g in self.groups:
                for row in g.spec.rows:
                    g.storage[row.name] = torch.zeros((len(g.runs), self.num_pages) + row.page_shape(page_size),
                                                      dtype=row.dtype or dtype, device=self.device)
        self._state_tensors: List[Optional[torch.Tensor]] = []
        for i, p in enumerate(plans):
            slot = LayerSlot()
            src = p.cache_from if p.cache_from is not None else i
            if src in owner_index:
                gid, idx = owner_index[src]
                slot.group = gid
                slot.writes = p.cache_from is None
                slot.page_size = page_size
                slot.rows = {name: t[idx] for name, t in self.groups[gid].storage.items()}
            if p.state is not None and allocate:
                # one row beyond the request slots: the state of the padding rows of a captured step, which no live
                # request ever holds (a mixer may read and write it like any other row)
                slot.state = torch.zeros((max_requests + 1,) + tuple(p.state.shape), dtype=p.state.dtype, device=self.device)
            self._state_tensors.append(slot.state)
            self.slots.append(slot)
        self._free_state = list(range(max_requests - 1, -1, -1))
        self.padding_state_slot = max_requests
        for g in self.groups:
            g.tables = TableArena(max_requests)
        self.requests: Dict[object, RequestCache] = {}
        self.pages_given_back_by_window = 0
        self.sharing_refused = ""
        if prefix_share and any(g.spec.window > 0 for g in self.groups):
            self.sharing_refused = "a group of layers has a window"
        elif prefix_share and any(p.state is not None for p in plans):
            self.sharing_refused = "a layer keeps per-request state"
        elif prefix_share and not self.groups:
            self.sharing_refused = "no layer owns pages"
        self.tree: Optional[PrefixTree] = PrefixTree(page_size) if prefix_share and not self.sharing_refused else None
        self.copies_on_write = 0

    # ------------------------------------------------------------------------------------------ requests

    def open(self, rid) -> RequestCache:
        if rid in self.requests:
            raise ValueError(f"request {rid!r} already holds a cache")
        if not self._free_state:
            raise OutOfPages(f"all {self.max_requests} request slots are in use")
        slot = self._free_state.pop()
        rc = RequestCache(rid, 0, slot, [g.tables.table(slot) for g in self.groups], [0 for _ in self.groups])
        for t in self._state_tensors:
            if t is not None:
                t[rc.state_slot].zero_()
        self.requests[rid] = rc
        return rc

    def has(self, rid) -> bool:
        return rid in self.requests

    def group_index(self, spec: PageSpec) -> int:
        """The group that holds the layer runs with this page spec (a step planner finds its block tables by it)."""
        for g in self.groups:
            if g.spec == spec:
                return g.gid
        raise KeyError(f"no group of layer runs has the page spec {spec}")

    def length(self, rid) -> int:
        return self.requests[rid].length

    def close(self, rid) -> None:
        """Gives back every page and the state slot of a request (finish, abort or preemption)."""
        rc = self.requests.pop(rid)
        for g, table in zip(self.groups, rc.tables):
            for p in table:
                if p >= 0:
                    g.pool.release(p)
        for node in rc.path:  # the tree keeps its own reference: these pages stay as cache
            self.tree.unuse(node)
        for table in rc.tables:
            table.clear()
        self._free_state.append(rc.state_slot)

    # ------------------------------------------------------------------------------------------ pages

    def _first_needed(self, g: KvGroup, length: int) -> int:
        """The oldest position any query at position >= length still sees in group g."""
        return max(0, length + 1 - g.spec.window) if g.spec.window > 0 else 0

    def pages_needed(self, rid, n: int) -> List[int]:
        """Pages each group would have to allocate for the next n tokens of the request."""
        rc = self.requests.get(rid)
        length = rc.length if rc else 0
        out = []
        for gi, g in enumerate(self.groups):
            have = len(rc.tables[gi]) if rc else 0
            out.append(max(0, -(-(length + n) // self.page_size) - have))
        return out

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def free_pages(self) -> List[int]:
        """Pages each group can still hand out: the free ones and those that only the prefix tree holds."""
        idle = self.tree.idle if self.tree else 0
        return [g.pool.free_pages + idle for g in self.groups]

    def _alloc(self, gi: int) -> int:
        """A page of group gi; when none is free, the cached page used longest ago makes room (in every group:
        a tree node holds one page of each)."""
        while True:
            try:
                return self.groups[gi].pool.alloc()
            except OutOfPages:
                node = self.tree.pop_evictable() if self.tree else None
                if node is None:
                    raise
                for g, p in zip(self.groups, node.pages):
                    g.pool.release(p)

    def begin_write(self, rid, n: int) -> int:
        """Makes room for positions [length, length + n) in every group; returns ``length``.

        Either every group gets its pages or none does: on OutOfPages the pages this call took are returned
        before the error leaves (kv/KvSequence.java:116-146 extends one table; here there may be several).
        """
        if n < 0:
            raise ValueError("negative token count")
        rc = self.requests[rid]
        need = -(-(rc.length + n) // self.page_size)
        taken: List[Tuple[int, int]] = []
        if n > 0 and rc.length % self.page_size and rc.length // self.page_size < len(rc.path):
            self._own_boundary_page(rc)
        try:
            for gi, g in enumerate(self.groups):
                while len(rc.tables[gi]) < need:
                    p = self._alloc(gi)
                    rc.tables[gi].append(p)
                    taken.append((gi, p))
        except OutOfPages:
            for gi, p in reversed(taken):
                popped = rc.tables[gi].pop()
                assert popped == p
                self.groups[gi].pool.release(p)
            raise
        return rc.length

    def _own_boundary_page(self, rc: RequestCache) -> None:
        """The next write lands inside a published page (the request was cut back into it): the rows kept move
        to a page of the request's own and the published one is left as it is (kv/KvSequence.java:116-146)."""
        B = self.page_size
        bi, rows = rc.length // B, rc.length % B
        node = rc.path[bi]
        fresh: List[int] = []
        try:
            for gi in range(len(self.groups)):
                fresh.append(self._alloc(gi))  # the node is in use by this request, so it is not evicted
        except OutOfPages:
            for gi, p in enumerate(fresh):
                self.groups[gi].pool.release(p)
            raise
        for gi, g in enumerate(self.groups):
            self._copy(gi, node.pages[gi], fresh[gi], rows)
            rc.tables[gi][bi] = fresh[gi]
            g.pool.release(node.pages[gi])
        for later in rc.path[bi:]:
            self.tree.unuse(later)
        del rc.path[bi:]
        self.copies_on_write += 1

    def _copy(self, gi: int, src: int, dst: int, rows: int) -> None:
        if rows > 0:
            self.copy_page(gi, src, dst, rows)

    def rollback_write(self, rid) -> None:
        """Undoes a ``begin_write`` whose step did not run: pages beyond the held length go back."""
        rc = self.requests[rid]
        keep = -(-rc.length // self.page_size)
        for gi, g in enumerate(self.groups):
            while len(rc.tables[gi]) > keep:
                p = rc.tables[gi].pop()
                if p >= 0:
                    g.pool.release(p)

    def commit(self, rid, n: int) -> None:
        """The step wrote n positions: advance the length and give back pages a window has passed."""
        rc = self.requests[rid]
        rc.length += n
        assert all(len(t) * self.page_size >= rc.length for t in rc.tables), "commit beyond the pages begun"
        for gi, g in enumerate(self.groups):
            if g.spec.window <= 0:
                continue
            first = self._first_needed(g, rc.length)
            whole = first // self.page_size  # table entries wholly before `first`
            for b in range(rc.released[gi], whole):
                p = rc.tables[gi][b]
                if p >= 0:
                    g.pool.release(p)
                    rc.tables[gi][b] = -1
                    self.pages_given_back_by_window += 1
            rc.released[gi] = max(rc.released[gi], whole)

    def truncate(self, rid, length: int) -> None:
        """Forgets positions >= length (kv/KvSequence.java:149-167). A group that already gave pages of the
        kept range back cannot do it, and neither can a request with per-request state."""
        rc = self.requests[rid]
        if length > rc.length or length < 0:
            raise ValueError(f"cannot truncate {rc.length} positions to {length}")
        if length < rc.length and any(t is not None for t in self._state_tensors):
            raise ValueError("a model with per-request state cannot be rewound")
        keep = -(-length // self.page_size)
        for gi, g in enumerate(self.groups):
            if g.spec.window > 0 and self._first_needed(g, length) < rc.released[gi] * self.page_size:
                raise ValueError("the window of this group has already given back pages the shorter sequence needs")
            while len(rc.tables[gi]) > keep:
                p = rc.tables[gi].pop()
                if p >= 0:
                    g.pool.release(p)
        for node in rc.path[keep:]:
            self.tree.unuse(node)
        del rc.path[keep:]
        rc.length = length

    # ------------------------------------------------------------------------------------------ sharing

    @property
    def sharing(self) -> bool:
        return self.tree is not None

    def match(self, tokens: Sequence[int], limit: Optional[int] = None) -> PrefixMatch:
        """How much of tokens[0 : limit) the tree holds; nothing changes hands (kv/KvPool.java:375-415)."""
        if self.tree is None:
            return PrefixMatch()
        return self.tree.match(tokens, len(tokens) if limit is None else min(limit, len(tokens)))

    def adopt(self, rid, tokens: Sequence[int], n: int) -> int:
        """Makes a request that holds nothing yet start with the tree's pages for tokens[0 : n): full pages are
        shared, a last part that is only the start of a published page is copied into a page of the request's
        own. Returns the positions held now (fewer than n when the tree no longer has them or no page is free
        for the copy) (kv/KvPool.java:418-524)."""
        rc = self.requests[rid]
        if self.tree is None or n <= 0:
            return 0
        if rc.length or any(rc.tables):
            raise ValueError(f"request {rid!r} already holds positions; only a fresh request adopts a prefix")
        tree, B = self.tree, self.page_size
        t = tree.tick()
        node, got = tree.root, 0
        while got + B <= n:
            c = tree.child(node, tokens, got)
            if c is None:
                break
            tree.touch(c, t)
            tree.use(c)
            for gi, g in enumerate(self.groups):
                g.pool.retain(c.pages[gi])
                rc.tables[gi].append(c.pages[gi])
            rc.path.append(c)
            node = c
            got += B
        rows, c = tree.best_partial(node, tokens, got, min(B, n - got))
        if rows > 0:
            tree.touch(c, t)
            tree.use(c)  # the allocation below may evict: keep the source
            fresh: List[int] = []
            try:
                for gi in range(len(self.groups)):
                    fresh.append(self._alloc(gi))
                for gi in range(len(self.groups)):
                    self._copy(gi, c.pages[gi], fresh[gi], rows)
                    rc.tables[gi].append(fresh[gi])
                got += rows
                self.copies_on_write += 1
            except OutOfPages:
                for gi, p in enumerate(fresh):
                    self.groups[gi].pool.release(p)
            finally:
                tree.unuse(c)
        rc.length = got
        if got:
            tree.hits += 1
            tree.hit_tokens += got
        return got

    def published_pages(self, rid) -> int:
        return len(self.requests[rid].path)

    def publish(self, rid, tokens: Sequence[int]) -> None:
        """Makes the full pages that hold tokens[0 : n), n = min(len(tokens), positions held), nodes of the tree.
        Where the tree already has a page for the same tokens the request switches to it and its own copy goes
        back to the pool (kv/KvPool.java:554-587). ``tokens`` must be what the request's positions were
        computed from."""
        if self.tree is None:
            return
        rc = self.requests[rid]
        tree, B = self.tree, self.page_size
        full = min(len(tokens), rc.length) // B
        if full <= len(rc.path):
            return
        t = tree.tick()
        node = rc.path[-1] if rc.path else tree.root
        for i in range(len(rc.path), full):
            key = tuple(int(x) for x in tokens[i * B:(i + 1) * B])
            c = node.kids.get(key)
            if c is not None:
                tree.touch(c, t)
                tree.use(c)
                for gi, g in enumerate(self.groups):
                    g.pool.retain(c.pages[gi])
                    g.pool.release(rc.tables[gi][i])
                    rc.tables[gi][i] = c.pages[gi]
                tree.dedups += 1
            else:
                pages = [rc.tables[gi][i] for gi in range(len(self.groups))]
                for gi, g in enumerate(self.groups):
                    g.pool.retain(pages[gi])  # the tree's reference
                c = tree.attach(node, key, pages)
                tree.use(c)
            rc.path.append(c)
            node = c

    def drop_cached(self) -> int:
        """Evicts every page that only the tree holds; returns how many nodes went."""
        n = 0
        while self.tree is not None:
            node = self.tree.pop_evictable()
            if node is None:
                break
            for g, p in zip(self.groups, node.pages):
                g.pool.release(p)
            n += 1
        return n

    # ------------------------------------------------------------------------------------------ step views

    def slot_indices(self, rid, gi: int, start: int, n: int) -> List[int]:
        """page * page_size + offset for positions [start, start + n) of the request in group gi."""
        t = self.requests[rid].tables[gi]
        B = self.page_size
        out = []
        for p in range(start, start + n):
            page = t[p // B]
            assert page >= 0, "writing into a page that was given back"
            out.append(page * B + (p % B))
        return out

    def table(self, rid, gi: int) -> List[int]:
        return self.requests[rid].tables[gi]

    def copy_page(self, gi: int, src: int, dst: int, rows: int) -> None:
        """Copies the first ``rows`` positions of one page to another in every layer run of group ``gi`` (the
        reference's KvStorage.copy, kv/KvStorage.java:43: what a copy-on-write of a shared, partly filled page does)."""
        from ..kernels import ops
        g = self.groups[gi]
        if g.pool.refs(src) <= 0 or g.pool.refs(dst) <= 0:
            raise ValueError("both pages of a copy must be held")
        for row in g.spec.rows:  # none when the manager only keeps books (host-side tests)
            t = g.storage.get(row.name)
            if t is None:
                continue
            a = row.position_axis
            outer = 1
            for d in row.shape[:a]:
                outer *= d
            inner = 1
            for d in row.shape[a:]:
                inner *= d
            ops.copy_page_rows(t.view(t.shape[0], t.shape[1], outer, self.page_size, inner), src, dst, rows)

    def stats(self) -> dict:
        return {
            "page_size": self.page_size,
            "groups": [{"runs": len(g.runs), "window": g.spec.window, "pages": g.pool.num_pages,
                        "used": g.pool.used_pages, "free": g.pool.free_pages, "high_water": g.pool.high_water,
                        "allocations": g.pool.allocations} for g in self.groups],
            "requests": len(self.requests),
            "state_slots_free": len(self._free_state),
            "window_pages_given_back": self.pages_given_back_by_window,
            "prefix": None if self.tree is None else {
                "nodes": self.tree.nodes, "idle": self.tree.idle, "hits": self.tree.hits,
                "hit_tokens": self.tree.hit_tokens, "evictions": self.tree.evictions, "dedups": self.tree.dedups,
                "copies_on_write": self.copies_on_write},
        }

    def check(self) -> None:
        """No page lost, held twice or freed twice: a page's references are the live tables it is in plus the
        prefix tree's one; a page in two tables is a node of the tree and at the same place in both."""
        nodes = list(self.tree.walk()) if self.tree else []
        users = {id(n): 0 for n in nodes}
        for rc in self.requests.values():
            for i, node in enumerate(rc.path):
                assert node.attached and id(node) in users, f"request {rc.rid!r} goes through a node that left the tree"
                assert node.parent is (rc.path[i - 1] if i else self.tree.root)
                users[id(node)] += 1
                for gi in range(len(self.groups)):
                    assert rc.tables[gi][i] == node.pages[gi], "a table and its tree path name different pages"
        for n in nodes:
            assert n.users == users[id(n)], f"node {n.nid}: {n.users} users counted, {users[id(n)]} tables go through it"
            assert n.users == 0 or n.parent is self.tree.root or n.parent.users >= n.users
        if self.tree:
            assert self.tree.nodes == len(nodes) and self.tree.idle == sum(1 for n in nodes if n.users == 0)
        for gi, g in enumerate(self.groups):
            g.pool.check()
            expect: Dict[int, int] = {}
            for n in nodes:
                assert n.pages[gi] not in expect, f"page {n.pages[gi]} of group {gi} is two nodes of the tree"
                expect[n.pages[gi]] = 1
            for rc in self.requests.values():
                for i, p in enumerate(rc.tables[gi]):
                    if p < 0:
                        continue
                    if i >= len(rc.path):
                        assert p not in expect, f"page {p} of group {gi} is held twice (request {rc.rid!r})"
                    expect[p] = expect.get(p, 0) + 1
            for p, refs in expect.items():
                assert g.pool.refs(p) == refs, f"group {gi} page {p}: {g.pool.refs(p)} references, {refs} holders"
            assert len(expect) == g.pool.used_pages, f"group {gi}: {g.pool.used_pages} pages held, {len(expect)} accounted for"
        slots = [rc.state_slot for rc in self.requests.values()]
        assert len(set(slots)) == len(slots) and not (set(slots) & set(self._free_state))
        assert len(slots) + len(self._free_state) == self.max_requests
