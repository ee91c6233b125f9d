"""The cache manager: paged keys and values per group of layers, block tables per request, state slots.

What is kept of the reference's design (docs/24-paged-kv-cache.md:53-72; kv/KvSequence.java:116-146): a
page holds ``page_size`` consecutive positions of every layer of its group; the address of position p is
page ``table[p // page_size]``, row ``p % page_size``; before a step writes positions [pos, pos + n) the
table is extended to ceil((pos + n) / page_size) entries.

What is different: the reference has one group and refuses models whose layers differ
(model/Decoder.java:40-49). Here every cache-owning run of the layer schedule declares a ``KvSpec``;
runs with equal specs form a group with its own pool, storage and block table per request. A group with
a window gives pages back as soon as every position in them is older than any later query can see
(model/Attention.java:68-71: the query at p sees keys from max(0, p + 1 - window)). Beside the pages
there are fixed-size state slots: one index per live request into per-run state tensors.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .pages import OutOfPages, PagePool


@dataclass(frozen=True)
class KvSpec:
    """What one cache-owning layer run stores per position."""

    kv_heads: int
    head_dim: int
    window: int = 0  # 0 = all earlier keys stay visible


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size that one layer run keeps (shape without the slot dimension)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class CacheEntryPlan:
    """One run of the layer schedule as the cache manager sees it."""

    kv: Optional[KvSpec] = None  # None: this run owns no pages
    cache_from: Optional[int] = None  # reads the pages of that earlier run
    state: Optional[StateSpec] = None


@dataclass
class LayerSlot:
    """What one run of the schedule is handed at every step."""

    group: Optional[int] = None
    k_cache: Optional[torch.Tensor] = None  # [pages, kv_heads, page_size, head_dim]
    v_cache: Optional[torch.Tensor] = None
    writes: bool = True
    state: Optional[torch.Tensor] = None  # [slots, *shape]


class KvGroup:
    def __init__(self, gid: int, spec: KvSpec, runs: List[int], num_pages: int, page_size: int):
        self.gid = gid
        self.spec = spec
        self.runs = runs
        self.pool = PagePool(num_pages, page_size)
        self.storage: Optional[torch.Tensor] = None  # [len(runs), 2, pages, kv_heads, page_size, head_dim]


@dataclass
class RequestCache:
    rid: object
    length: int = 0  # positions held
    state_slot: int = -1
    tables: List[List[int]] = field(default_factory=list)  # per group: page ids, -1 = given back
    released: List[int] = field(default_factory=list)  # per group: leading table entries already given back


class CacheManager:
    def __init__(self, plans: Sequence[CacheEntryPlan], page_size: int, pool_tokens: int, max_requests: int,
                 dtype: torch.dtype = torch.float32, device="cpu", allocate: bool = True):
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
                g.storage = torch.zeros((len(g.runs), 2, self.num_pages, g.spec.kv_heads, page_size, g.spec.head_dim),
                                        dtype=dtype, device=self.device)
        self._state_tensors: List[Optional[torch.Tensor]] = []
        for i, p in enumerate(plans):
            slot = LayerSlot()
            src = p.cache_from if p.cache_from is not None else i
            if src in owner_index:
                gid, idx = owner_index[src]
                slot.group = gid
                slot.writes = p.cache_from is None
                if allocate:
                    slot.k_cache = self.groups[gid].storage[idx, 0]
                    slot.v_cache = self.groups[gid].storage[idx, 1]
            if p.state is not None and allocate:
                slot.state = torch.zeros((max_requests,) + tuple(p.state.shape), dtype=p.state.dtype, device=self.device)
            self._state_tensors.append(slot.state)
            self.slots.append(slot)
        self._free_state = list(range(max_requests - 1, -1, -1))
        self.requests: Dict[object, RequestCache] = {}
        self.pages_given_back_by_window = 0

    # ------------------------------------------------------------------------------------------ requests

    def open(self, rid) -> RequestCache:
        if rid in self.requests:
            raise ValueError(f"request {rid!r} already holds a cache")
        if not self._free_state:
            raise OutOfPages(f"all {self.max_requests} request slots are in use")
        rc = RequestCache(rid, 0, self._free_state.pop(), [[] for _ in self.groups], [0 for _ in self.groups])
        for t in self._state_tensors:
            if t is not None:
                t[rc.state_slot].zero_()
        self.requests[rid] = rc
        return rc

    def has(self, rid) -> bool:
        return rid in self.requests

    def length(self, rid) -> int:
        return self.requests[rid].length

    def close(self, rid) -> None:
        """Gives back every page and the state slot of a request (finish, abort or preemption)."""
        rc = self.requests.pop(rid)
        for g, table in zip(self.groups, rc.tables):
            for p in table:
                if p >= 0:
                    g.pool.release(p)
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
        return [g.pool.free_pages for g in self.groups]

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
        try:
            for gi, g in enumerate(self.groups):
                while len(rc.tables[gi]) < need:
                    p = g.pool.alloc()
                    rc.tables[gi].append(p)
                    taken.append((gi, p))
        except OutOfPages:
            for gi, p in reversed(taken):
                popped = rc.tables[gi].pop()
                assert popped == p
                self.groups[gi].pool.release(p)
            raise
        return rc.length

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
        rc.length = length

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
        ops.copy_page_rows(g.storage, src, dst, rows)

    def stats(self) -> dict:
        return {
            "page_size": self.page_size,
            "groups": [{"runs": len(g.runs), "window": g.spec.window, "pages": g.pool.num_pages,
                        "used": g.pool.used_pages, "free": g.pool.free_pages, "high_water": g.pool.high_water,
                        "allocations": g.pool.allocations} for g in self.groups],
            "requests": len(self.requests),
            "state_slots_free": len(self._free_state),
            "window_pages_given_back": self.pages_given_back_by_window,
        }

    def check(self) -> None:
        """No page lost, held twice or freed twice: every held page is in exactly one live table."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            seen = {}
            for rc in self.requests.values():
                for p in rc.tables[gi]:
                    if p < 0:
                        continue
                    assert p not in seen, f"page {p} of group {gi} is in the tables of {seen[p]!r} and {rc.rid!r}"
                    seen[p] = rc.rid
                    assert g.pool.refs(p) == 1
            assert len(seen) == g.pool.used_pages, f"group {gi}: {g.pool.used_pages} pages held, {len(seen)} in tables"
        slots = [rc.state_slot for rc in self.requests.values()]
        assert len(set(slots)) == len(slots) and not (set(slots) & set(self._free_state))
        assert len(slots) + len(self._free_state) == self.max_requests
