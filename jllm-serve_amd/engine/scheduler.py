"""The scheduler: admission, cutting prompts into portions under a token budget, decoding, preemption.

Policy kept from the reference's pass planner (engine/PassPlanner.java:74-112): the single rows of decoding
requests ("riders") go first, by arrival, each while it fits the budget; prompt portions take what is
left, a portion being trimmed to the leftover only if that is at least ``min_chunk`` rows (or the whole
remainder when that is smaller), else it waits for a pass with more room; when nothing fits, the oldest
item goes alone, trimmed to the budget, so a pass is never empty while work is pending. Unlike the
reference (one chunk per pass, docs/25-scheduler.md:379) a pass may carry portions of several prompts.
A prompt is cut into portions of at most ``prefill_chunk`` tokens (engine/Engine.java:557-608: chunks of
``backend.batch``).

Admission (engine/Admission.java:217-285): first come, first served within a class, while
fewer than ``max_running`` requests run and the pool has the pages the first portion needs. When the cache
shares prefixes, a request that is admitted takes over the pages the prefix tree holds for the start of its
tokens, and only the rest is computed; at least its last token always is, since its logits are needed
(engine/Engine.java:518-521). After every pass the full pages a request has computed are published
(engine/Engine.java:568-571, :773-780), so a preempted request finds its own pages again if nothing evicted
them meanwhile.

Classes (engine/Admission.java:192-214, :262-301; engine/PassPlanner.java:60-100): a request is interactive (0)
or background (1); its effective class falls by one for every ``age_promote_s`` it has waited, so background
work is never starved. Waiting requests are admitted by effective class, then arrival; rows of a pass are
given in the same order; a background portion is capped at ``background_chunk_cap`` rows while an interactive
request decodes in the same pass; when every place is taken and an interactive request waits, the background
request that started last is preempted (the reference pauses it and recomputes what it cannot bring back).
Within a class a preempted request comes before new ones, then the highest score wins: tokens of the request
that the prefix tree holds + 2000 per second waited (engine/Admission.java:59, :222-238), then the oldest.
Sessions (engine/Admission.java:184-189, :225; ``engine.session-max-running``): a request may name a session; a session
that already has ``session_max_running`` requests running waits, although places are free, until one of them ends.

When pages run out (the reference raises KvPoolExhausted to the request, kv/KvPool.java:257-267, or
suspends a background slot and recomputes what it lost, docs/25-scheduler.md:195-215): nothing new is
admitted; if a running request cannot get the pages of its next rows, the request admitted last (a
background one before an interactive one) is preempted: its pages and state slot go back, it returns to the head of the waiting queue and its prompt
and the tokens generated so far are computed again later. A request that is alone and still does not fit
ends with finish reason "length": the pool is its context limit.
"""
from __future__ import annotations

import collections
import itertools
import time
from dataclasses import dataclass, field
from typing import Any, Deque, Dict, List, Optional, Sequence

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class SchedulerConfig:
    max_batch_tokens: int = 2048  # rows per pass (engine.pass-budget; 0 = prefill_chunk + mixed_reserve)
    prefill_chunk: int = 2048  # most rows of one prompt in a pass (backend.batch)
    max_running: int = 64  # engine.max-running (0 = as many as there are state slots)
    min_chunk: int = 16  # ModelLoader.java:451-454
    max_positions: int = 4096  # context limit per request (backend.ctx)
    age_promote_s: float = 10.0  # engine.age-promote-ms: a class is worth this much waiting; 0 = classes never age
    background_chunk_cap: int = 0  # engine.background-chunk-cap: rows of a background portion beside an interactive rider; 0 = no cap
    preempt: bool = True  # engine.preempt: an interactive arrival may displace a running background request
    session_max_running: int = 0  # engine.session-max-running: most requests of one session running at once; 0 = no limit

    def __post_init__(self):
        if self.max_batch_tokens < 1:
            raise ValueError("a pass needs a budget of at least one row")  # PassPlanner.java:50-54
        if self.prefill_chunk < 1 or self.min_chunk < 1 or self.max_running < 0:
            raise ValueError("prefill_chunk and min_chunk must be positive, max_running not negative")


@dataclass
class Request:
    rid: Any
    prompt: List[int]
    params: Any
    arrival: int
    output: List[int] = field(default_factory=list)
    logprobs: list = field(default_factory=list)  # one entry per output token when the request asked for them
    prompt_logprobs: list = field(default_factory=list)  # one entry per prompt token (the first is None) when asked for
    computed: int = 0  # tokens of (prompt + output) whose keys and values are in the cache
    status: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0
    sampler: Any = None
    stats: Dict[str, float] = field(default_factory=dict)
    cancelled: bool = False
    last_pass: int = -1
    cached_tokens: int = 0  # positions taken over from the prefix tree instead of computed (all admissions)
    priority: int = 0  # 0 interactive, 1 background (engine/Priority.java)
    enqueued: float = 0.0  # the scheduler's clock when the request arrived
    admitted: int = -1  # order of admission; the latest is the first to be displaced
    unread: int = 0  # 1: a token was sampled on the device and is not in ``output`` yet (the engine's lookahead)
    session: Optional[str] = None  # the request's session (the reference's OpenAI ``user``); None = none

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def pending(self) -> int:
        """Tokens not yet in the cache; the last sampled token is among them until the next step feeds it
        (engine/Engine.java:771-781)."""
        return len(self.prompt) + len(self.output) + self.unread - self.computed


@dataclass
class Planned:
    request: Request
    n: int  # rows of this request in the pass
    wants_logits: bool  # the portion reaches the end of the known tokens


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache, clock=time.monotonic):
        self.config = config
        self.cache = cache
        self.clock = clock
        self._admissions = itertools.count()
        self.displaced = 0  # background requests preempted for an interactive arrival
        self.waiting: Deque[Request] = collections.deque()
        self.running: List[Request] = []
        self._arrivals = itertools.count()
        self.preemptions = 0
        self.passes = 0
        self.rows = 0
        self.ledger: Optional[list] = None  # a list here makes count_pass keep every pass's work (measurements)

    # ------------------------------------------------------------------------------------------ queue

    def add(self, rid, prompt: Sequence[int], params, sampler=None, priority: int = 0, session: Optional[str] = None) -> Request:
        prompt = list(prompt)
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if len(prompt) >= self.config.max_positions:  # engine/Engine.java:505-507
            raise ValueError(f"prompt of {len(prompt)} tokens does not fit the context of {self.config.max_positions}")
        capacity = min(g.pool.num_pages for g in self.cache.groups) * self.cache.page_size if self.cache.groups else None
        if capacity is not None and len(prompt) + 1 > capacity:
            raise ValueError(f"prompt of {len(prompt)} tokens can never fit the KV pool of {capacity} positions")
        if priority not in (0, 1):
            raise ValueError(f"priority must be 0 (interactive) or 1 (background), got {priority!r}")
        r = Request(rid, prompt, params, next(self._arrivals), sampler=sampler, priority=priority, enqueued=self.clock(),
                    session=session)
        self.waiting.append(r)
        return r

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def rank(self, r: Request, now: Optional[float] = None) -> int:
        """The request's class now: lowered by one per ``age_promote_s`` waited, not below 0 (PassPlanner.java:60-67)."""
        age = self.config.age_promote_s
        if age <= 0 or r.priority == 0:
            return r.priority
        now = self.clock() if now is None else now
        return max(0, r.priority - int(max(0.0, now - r.enqueued) // age))

    AGING_TOKENS_PER_SECOND = 2000.0  # engine/Admission.java:59
    SCORED_WAITERS = 32  # requests (by arrival) whose cached prefix is looked up when the next one is chosen

    def _admissible(self) -> List[Request]:
        """The waiting requests whose session is under its limit (engine/Admission.java:183-189, :225: a session that
        holds ``session_max_running`` places waits although places are free; another session does not). A place is
        held by a running request and, as the reference counts its paused slots, by a request that was preempted and
        waits to go on: that one is admissible itself (it holds its place already), a new request of its session
        is not."""
        cap = self.config.session_max_running
        if cap <= 0:
            return list(self.waiting)
        holding: Dict[str, int] = {}
        for q in list(self.running) + [w for w in self.waiting if w.preemptions > 0]:
            if q.session is not None:
                holding[q.session] = holding.get(q.session, 0) + 1
        return [r for r in self.waiting if r.session is None or r.preemptions > 0 or holding.get(r.session, 0) < cap]

    def _next_waiting(self, now: float, among: Optional[List[Request]] = None) -> Request:
        """Who is admitted next (engine/Admission.java:222-238)."""
        among = list(self.waiting) if among is None else among
        hits = {}
        if self.cache.sharing and len(among) > 1:
            for r in sorted(among, key=lambda r: r.arrival)[:self.SCORED_WAITERS]:
                if not (getattr(r.params, "prompt_logprobs", False) and len(r.prompt_logprobs) < len(r.prompt)):
                    tokens = r.tokens
                    hits[id(r)] = self.cache.match(tokens, len(tokens) - 1).tokens

        def key(r: Request):
            score = hits.get(id(r), 0) + self.AGING_TOKENS_PER_SECOND * max(0.0, now - r.enqueued)
            return (self.rank(r, now), r.preemptions == 0, -score, r.arrival)
        return min(among, key=key)

    def _coming_prefix(self, tokens: List[int], rank: int, now: float) -> int:
        """Leading tokens of ``tokens`` that a running request still computing its prompt will have published when
        it is done: what arrives together and starts alike is computed once. Nobody waits for a request of a lower
        class: its portions may be held back by the very class that would be waiting."""
        B = self.cache.page_size
        best = 0
        for q in self.running:
            if q.computed >= len(q.prompt) or self.rank(q, now) > rank:
                continue
            n = min(len(q.prompt), len(tokens) - 1)
            same = 0
            while same < n and q.prompt[same] == tokens[same]:
                same += 1
            best = max(best, same // B * B)
        return best

    def _admit(self, r: Request) -> None:
        self.waiting.remove(r)
        r.status = RUNNING
        r.admitted = next(self._admissions)
        self.running.append(r)

    def _victim(self, now: float) -> Request:
        """Who gives way when pages run out: a background request before an interactive one, the one admitted last."""
        return max(self.running, key=lambda r: (self.rank(r, now), r.admitted))

    def limit(self, r: Request) -> int:
        """Most tokens the request may generate: min(max_tokens, ctx - prompt) (engine/Engine.java:619)."""
        return min(r.params.max_tokens, self.config.max_positions - len(r.prompt))

    # ------------------------------------------------------------------------------------------ planning

    def plan(self) -> List[Planned]:
        """Chooses the rows of the next pass and makes sure the cache can take them, preempting when a
        running request cannot get its pages. Returns [] only when nothing is pending."""
        while True:
            picks = self._pick()
            if not picks:
                return []
            short = self._first_short_of_pages(picks)
            if short is None:
                for p in picks:
                    p.request.last_pass = self.passes
                self.count_pass([(p.n, p.request.computed) for p in picks])
                return picks
            victim = self._victim(self.clock())
            if victim is short.request and len(self.running) == 1:
                # alone and still no room: the pool is this request's context limit
                self.finish(victim, "length")
                continue
            self.preempt(victim)

    def count_pass(self, rows_and_starts) -> None:
        """Books one pass: [(rows, position of the first)] per request. With ``ledger`` set to a list, every pass also
        leaves (requests with one row, keys those rows attend over, rows of portions, (row, key) pairs of portions):
        what a measurement needs to say how many bytes and flops the passes had to move."""
        self.passes += 1
        self.rows += sum(n for n, _ in rows_and_starts)
        if self.ledger is not None:
            ones = [(n, p) for n, p in rows_and_starts if n == 1]
            more = [(n, p) for n, p in rows_and_starts if n > 1]
            self.ledger.append((len(ones), sum(p + 1 for _, p in ones), sum(n for n, _ in more),
                                sum(n * p + n * (n + 1) // 2 for n, p in more)))

    def _pick(self) -> List[Planned]:
        cfg = self.config
        budget = cfg.max_batch_tokens
        used = 0
        picks: List[Planned] = []
        now = self.clock()
        max_running = min(cfg.max_running or self.cache.max_requests, self.cache.max_requests)
        # every place is taken and an interactive request waits: the background request that started last gives
        # its place (Admission.java:262-270, :288-301) and is computed again when there is room
        while cfg.preempt and self.waiting and len(self.running) >= max_running:
            behind = [b for b in self.running if b.priority > 0]
            able = self._admissible()  # a request held back by its session's limit displaces nobody
            if not behind or not able or min(self.rank(r, now) for r in able) != 0:
                break
            self.preempt(max(behind, key=lambda b: b.admitted))
            self.displaced += 1
        riders = [r for r in self.running if r.pending == 1 and r.computed >= len(r.prompt)]
        chunks = [r for r in self.running if not (r.pending == 1 and r.computed >= len(r.prompt))]
        interactive_rider = False
        for r in sorted(riders, key=lambda r: (self.rank(r, now), r.last_pass, r.arrival)):  # by class, then whoever waited longest
            if used + 1 <= budget:
                picks.append(Planned(r, 1, True))
                used += 1
                interactive_rider |= self.rank(r, now) == 0
        free = list(self.cache.free_pages())
        for p in picks:
            for gi, need in enumerate(self.cache.pages_needed(p.request.rid, p.n)):
                free[gi] -= need

        def portion(pending: int, r: Optional[Request] = None) -> int:
            room = budget - used
            if r is not None and cfg.background_chunk_cap > 0 and interactive_rider and self.rank(r, now) > 0:
                room = min(room, cfg.background_chunk_cap)  # PassPlanner.java:94-96
            rows = min(pending, cfg.prefill_chunk, room)
            return rows if rows >= min(cfg.min_chunk, pending) and rows > 0 else 0

        for r in sorted(chunks, key=lambda r: (self.rank(r, now), r.arrival)):
            n = portion(r.pending, r)
            if n:
                picks.append(Planned(r, n, n == r.pending))
                used += n
                for gi, need in enumerate(self.cache.pages_needed(r.rid, n)):
                    free[gi] -= need
        # admission: by class, then first come first served, while places, budget and pages allow
        while self.waiting:
            if len(self.running) >= max_running:
                break
            able = self._admissible()
            if not able:
                break  # everybody who waits belongs to a session that holds its limit
            r = self._next_waiting(now, able)
            whole = getattr(r.params, "prompt_logprobs", False) and len(r.prompt_logprobs) < len(r.prompt)
            tokens = r.tokens if self.cache.sharing and not whole else None
            found = self.cache.match(tokens, len(tokens) - 1) if tokens is not None else None
            held = found.tokens if found else 0
            if found is not None and self._coming_prefix(tokens, self.rank(r, now), now) >= held + self.cache.page_size:
                break  # a running request is computing a longer start of these tokens: wait and take its pages over
            n = portion(r.pending - held, r)
            if not n:
                break
            if found and held:
                # shared pages are not allocated, but those nobody uses now stop being pages that could be evicted
                pages = self.cache.pages_for(held + n) - found.nodes + found.idle_nodes
                need = [pages] * len(free)
            else:
                need = self.cache.pages_needed(r.rid, n)
            if any(f - nd < 0 for f, nd in zip(free, need)):
                break
            self._admit(r)
            if found and held:
                self.cache.open(r.rid)
                r.computed = self.cache.adopt(r.rid, tokens, held)
                r.cached_tokens += r.computed
                n = portion(r.pending, r) or min(r.pending, max(1, budget - used))
            picks.append(Planned(r, n, n == r.pending))
            used += n
            for gi, nd in enumerate(need):
                free[gi] -= nd
        if not picks and (self.running or self.waiting):
            # nothing fits the budget as it is: the oldest goes alone, trimmed (PassPlanner.java:105-110)
            if self.running:
                r = min(self.running, key=lambda r: r.arrival)
            else:
                r = self._next_waiting(now)  # nothing runs: no session holds anything
                self._admit(r)
            n = min(r.pending, budget, cfg.prefill_chunk)
            picks.append(Planned(r, n, n == r.pending))
        # portions first so their rows start the batch, then the riders (PassPlanner.java:70-73)
        picks.sort(key=lambda p: (p.n == 1 and p.request.computed >= len(p.request.prompt), p.request.arrival))
        return picks

    def _first_short_of_pages(self, picks: List[Planned]) -> Optional[Planned]:
        free = list(self.cache.free_pages())
        for p in picks:
            need = self.cache.pages_needed(p.request.rid, p.n)
            for gi, nd in enumerate(need):
                free[gi] -= nd
            if any(f < 0 for f in free):
                return p
        return None

    # ------------------------------------------------------------------------------------------ outcomes

    def preempt(self, r: Request) -> None:
        """Frees everything the request holds and puts it back at the head of the queue; its prompt and the
        tokens generated so far are computed again when it is admitted next."""
        self.running.remove(r)
        if self.cache.has(r.rid):
            self.cache.close(r.rid)
        r.computed = 0
        r.status = WAITING
        r.preemptions += 1
        self.preemptions += 1
        self.waiting.appendleft(r)

    def computed(self, picks: Sequence[Planned]) -> None:
        """The pass ran: the picked rows are in the cache now, and pages they completed are published."""
        cache = self.cache
        for p in picks:
            r = p.request
            r.computed += p.n
            if cache.sharing and cache.has(r.rid) and r.computed // cache.page_size > cache.published_pages(r.rid):
                cache.publish(r.rid, r.tokens[:r.computed])

    def finish(self, r: Request, reason: str) -> None:
        if r in self.running:
            self.running.remove(r)
        elif r in self.waiting:
            self.waiting.remove(r)
        if self.cache.has(r.rid):
            self.cache.close(r.rid)
        r.status = FINISHED
        r.finish_reason = reason

    def stats(self) -> dict:
        return {"waiting": len(self.waiting), "running": len(self.running), "passes": self.passes, "rows": self.rows,
                "rows_per_pass": self.rows / self.passes if self.passes else 0.0, "preemptions": self.preemptions,
                "displaced": self.displaced}
