"""The prefix tree: full pages that requests have published, found again by the tokens that lead to them.

The reference's pool keeps a radix tree over blocks (kv/KvPool.java:375-415 ``match``, :418-524 ``adopt``,
:554-587 ``publish``; docs/24-paged-kv-cache.md:87-167): a node is one full block, reached from its parent by
the block's tokens; a published block is immutable; a block nobody references stays in the tree as cache
and is evicted, oldest use first and leaves before their parents, when the pool needs a page
(kv/KvPool.java:249-275, :327-351). A prompt may also share only the start of a block: then the rows are
copied into a page of the request's own.

Here a node holds one page per group of layers (all groups advance together). The tree owns one reference
to each of its pages; ``users`` counts the requests whose tables go through the node. This file is host
bookkeeping only: it never touches a pool or storage, the cache manager does.
"""
from __future__ import annotations

import heapq
import itertools
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple


class PrefixNode:
    __slots__ = ("parent", "tokens", "pages", "kids", "tick", "depth", "nid", "users", "attached")

    def __init__(self, parent: Optional["PrefixNode"], tokens: Tuple[int, ...], pages: List[int], nid: int):
        self.parent = parent
        self.tokens = tokens
        self.pages = pages  # one page id per group
        self.kids: Dict[Tuple[int, ...], "PrefixNode"] = {}
        self.tick = 0
        self.depth = parent.depth + 1 if parent is not None else 0
        self.nid = nid
        self.users = 0
        self.attached = True


@dataclass(frozen=True)
class PrefixMatch:
    tokens: int = 0  # leading tokens the tree holds, to the token
    nodes: int = 0  # full pages among them
    idle_nodes: int = 0  # of those, pages nobody uses now (adopting them takes them out of what can be evicted)
    partial: int = 0  # rows of one more page that would be copied


class PrefixTree:
    def __init__(self, page_size: int):
        self.page_size = page_size
        self.root = PrefixNode(None, (), [], 0)
        self._ids = itertools.count(1)
        self._tick = 0
        self._heap: List[Tuple[int, int, int, PrefixNode]] = []  # (tick, -depth, id, node), entries may be stale
        self.nodes = 0
        self.idle = 0  # nodes with no user: what eviction may take
        self.evictions = 0
        self.dedups = 0
        self.hits = 0
        self.hit_tokens = 0

    # ------------------------------------------------------------------------------------------ use counts

    def tick(self) -> int:
        self._tick += 1
        return self._tick

    def touch(self, node: PrefixNode, t: int) -> None:
        if node.tick != t:
            node.tick = t
            if node.users == 0:
                self._push(node)

    def _push(self, node: PrefixNode) -> None:
        if len(self._heap) > 4 * self.nodes + 64:  # mostly stale entries: start again from the idle nodes
            self._heap = [(n.tick, -n.depth, n.nid, n) for n in self.walk() if n.users == 0 and n is not node]
            heapq.heapify(self._heap)
        heapq.heappush(self._heap, (node.tick, -node.depth, node.nid, node))

    def use(self, node: PrefixNode) -> None:
        if node.users == 0:
            self.idle -= 1
        node.users += 1

    def unuse(self, node: PrefixNode) -> None:
        assert node.users > 0
        node.users -= 1
        if node.users == 0:
            self.idle += 1
            self._push(node)

    # ------------------------------------------------------------------------------------------ the tree

    def child(self, node: PrefixNode, tokens: Sequence[int], off: int) -> Optional[PrefixNode]:
        return node.kids.get(tuple(tokens[off:off + self.page_size]))

    def best_partial(self, node: PrefixNode, tokens: Sequence[int], off: int, want: int) -> Tuple[int, Optional[PrefixNode]]:
        """Longest common start of tokens[off : off + want) with a child of ``node`` (kv/KvPool.java:418-438)."""
        best, found = 0, None
        if want <= 0:
            return 0, None
        for key, c in node.kids.items():
            k = 0
            while k < want and key[k] == tokens[off + k]:
                k += 1
            if k > best:
                best, found = k, c
        return best, found

    def match(self, tokens: Sequence[int], limit: int) -> PrefixMatch:
        """The longest prefix of tokens[0 : limit) that the tree holds (kv/KvPool.java:375-415)."""
        B = self.page_size
        t = self.tick()
        node, i, nodes, idle = self.root, 0, 0, 0
        while i + B <= limit:
            c = self.child(node, tokens, i)
            if c is None:
                break
            self.touch(c, t)
            nodes += 1
            idle += c.users == 0
            node = c
            i += B
        partial = 0
        if i < limit:
            partial, c = self.best_partial(node, tokens, i, min(B, limit - i))
            if c is not None:
                self.touch(c, t)
        return PrefixMatch(i + partial, nodes, idle, partial)

    def attach(self, parent: PrefixNode, tokens: Tuple[int, ...], pages: List[int]) -> PrefixNode:
        c = PrefixNode(parent, tokens, pages, next(self._ids))
        c.tick = self._tick
        parent.kids[tokens] = c
        self.nodes += 1
        self.idle += 1  # until its publisher calls use()
        return c

    def pop_evictable(self) -> Optional[PrefixNode]:
        """Detaches and returns the idle leaf used longest ago (ties: the deepest), or None. The caller frees
        its pages (kv/KvPool.java:327-351)."""
        while self._heap:
            tick, _, _, node = heapq.heappop(self._heap)
            if not node.attached or node.users or node.tick != tick or node.kids:
                continue  # stale entry; a node with children comes back when its last child goes
            parent = node.parent
            del parent.kids[node.tokens]
            node.attached = False
            self.nodes -= 1
            self.idle -= 1
            self.evictions += 1
            if parent is not self.root and parent.users == 0 and not parent.kids:
                self._push(parent)
            return node
        return None

    def walk(self):
        stack = list(self.root.kids.values())
        while stack:
            n = stack.pop()
            yield n
            stack.extend(n.kids.values())
