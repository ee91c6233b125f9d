"""The step function: one batch of (request, its next tokens) -> logits at the wanted places.

The reference's contract (model/Backend.java:131-153; cpu/CpuBackend.java:821-930): a pass holds one
segment per sequence, portions of prompts beside single decoded tokens; the rows of all segments form
one activation matrix; each segment is rotated at its own positions, stored into its own blocks and
attends over its own cache only; the final norm and the output head run over the selected rows only.
``beginWrite`` runs for every segment before any kernel (:853-857).

Here a step carries, for each request, the tokens that follow what its cache already holds (the position
of the first one is the cache's length) and the places among them whose logits are wanted. The ragged
batch becomes flat per-row arrays (token id, position, request index), per-group block tables and slot
indices, uploaded in one copy; then the model runs once over all rows.

The step function knows nothing of any mixer's kernels. A part that wants more about the batch on the device
or on the host (attention: its rows cut into tiles, whether every request brings one row) gives the model a
*step planner*: ``key`` (planners with equal keys plan once per step) and ``plan(StepBatch) -> StepPlan`` with
int32 arrays, which ride in the same upload, and host-side facts. Parts find their plan in ``step.plans[key]``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import host
from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages


@dataclass
class StepEntry:
    rid: Any
    tokens: Sequence[int]
    want: Sequence[int] = ()  # places among `tokens` whose logits are returned


@dataclass
class Segment:
    """One request's rows in the step (host side; parts that walk requests use it)."""

    rid: Any
    index: int  # request index in this step
    row0: int  # first row
    n: int
    pos0: int  # position of the first row
    state_slot: int


@dataclass
class GroupStep:
    block_table: torch.Tensor  # int32 [requests, width]
    slots: torch.Tensor  # int32 [rows]: page * page_size + offset where each row's per-position tensors go


@dataclass
class StepBatch:
    """What a step planner is told about the batch, on the host, before anything is uploaded."""

    segments: List[Segment]  # the live requests, in the order of their rows
    rows: int  # rows of the step; beyond the segments' rows: padding rows, one request each, that store nothing
    requests: int  # requests of the step, the padding ones included
    max_context: int  # positions the longest request holds after this step
    page_size: int
    cache: Any  # the cache manager, for planners that need block tables: cache.group_index(spec), cache.table(rid, group)
    padded: bool  # a step of fixed size (captured and replayed): a plan's arrays must then depend on rows and requests only


@dataclass
class StepPlan:
    """What one planner made of the batch: int32 arrays (uploaded with the rest of the step, handed back as device
    tensors) and facts that stay on the host."""

    arrays: Dict[str, Any] = field(default_factory=dict)  # name -> numpy int32 array (planner) / device tensor (parts)
    facts: Dict[str, Any] = field(default_factory=dict)


@dataclass
class StepContext:
    n_tokens: int
    n_requests: int
    token_ids: torch.Tensor  # int32 [rows]
    positions: torch.Tensor  # int32 [rows]
    row_req: torch.Tensor  # int32 [rows]: request index of each row
    state_slots: torch.Tensor  # int32 [requests]
    selected: torch.Tensor  # int32 [n_selected]: rows whose logits are wanted
    n_selected: int
    groups: List[GroupStep]
    segments: List[Segment]
    max_context: int = 1  # positions the longest request holds after this step (a captured step: of its bucket)
    plans: Dict[Any, StepPlan] = field(default_factory=dict)  # planner key -> what that planner made of this batch


class StepError(ValueError):
    pass


class ModelRunner:
    """Owns nothing but the wiring: the model's forward and the cache manager's bookkeeping around it."""

    def __init__(self, model, cache: CacheManager, max_positions: int):
        built_for = getattr(getattr(model, "build", None), "max_positions", None)
        if built_for is not None and max_positions > built_for:
            # the position encodings' tables have one row per position the model was built for; positions live on
            # the device, so no kernel could refuse a row beyond them
            raise ValueError(f"the runner would hold {max_positions} positions per request, the model was built for "
                             f"{built_for}: build the model with max_positions >= {max_positions}")
        self.model = model
        self.cache = cache
        self.max_positions = max_positions
        self.device = model.device
        self.vocab = model.config.vocab
        self.steps = 0
        self.rows = 0
        self.graphs = None  # captured decode steps (engine/graphs.py), when enabled
        self._planners = None

    # ------------------------------------------------------------------------------------------------

    def prepare(self, entries: Sequence[StepEntry]) -> StepContext:
        """Checks the entries, makes room in the cache for all of them (or for none) and builds the
        device-side description of the batch."""
        self.prepare_cache(entries)
        return self._describe(entries)

    def prepare_cache(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise StepError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            n = len(e.tokens)
            if n < 1:
                raise StepError(f"request {e.rid!r} brings no tokens")
            ids = np.asarray(e.tokens, dtype=np.int64)
            if ids.min() < 0 or ids.max() >= self.vocab:
                t = int(ids[(ids < 0) | (ids >= self.vocab)][0])
                raise StepError(f"request {e.rid!r}: token id {t} is outside the vocabulary of {self.vocab}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.rid!r}: wanted place {w} is outside its {n} tokens")
            held = self.cache.length(e.rid) if self.cache.has(e.rid) else 0
            if held + n > self.max_positions:
                raise StepError(f"request {e.rid!r} would hold {held + n} positions, the engine was built for {self.max_positions}")
        opened, begun = [], []
        try:
            for e in entries:
                if not self.cache.has(e.rid):
                    self.cache.open(e.rid)
                    opened.append(e.rid)
                self.cache.begin_write(e.rid, len(e.tokens))
                begun.append(e.rid)
        except OutOfPages:
            for rid in begun:
                if rid not in opened:
                    self.cache.rollback_write(rid)
            for rid in opened:
                self.cache.close(rid)
            raise

    def planners(self) -> list:
        """The model's step planners, one per distinct key (36 equal attention layers plan once)."""
        if self._planners is None:
            seen, out = set(), []
            for pl in (self.model.step_planners() if hasattr(self.model, "step_planners") else []):
                if pl.key not in seen:
                    seen.add(pl.key)
                    out.append(pl)
            self._planners = out
        return self._planners

    def _layout(self, entries: Sequence[StepEntry], pad_rows: int = 0, width: int = 0):
        """The batch as flat int32 arrays in a fixed order (token ids, positions, row -> request, state slots,
        selected rows, per group: slots, block table; then what the parts' planners add), plus the host-side
        segments.

        With ``pad_rows`` the arrays describe that many single-row requests: the extra ones read one key of
        page 0 and store nothing, so a captured step of a fixed size can run any smaller batch."""
        cache = self.cache
        B = cache.page_size
        n = len(entries)
        segments: List[Segment] = []
        counts, starts, state_slots, want_counts = [], [], [], []
        tokens: List[int] = []
        wants: List[int] = []
        row = 0
        for i, e in enumerate(entries):
            k = len(e.tokens)
            rc = cache.requests[e.rid]
            segments.append(Segment(e.rid, i, row, k, rc.length, rc.state_slot))
            counts.append(k)
            starts.append(rc.length)
            state_slots.append(rc.state_slot)
            want_counts.append(len(e.want))
            tokens.extend(e.tokens)
            wants.extend(e.want)
            row += k
        max_ctx = max([1] + [s.pos0 + s.n for s in segments])
        T = max(row, pad_rows)
        R = n + (T - row)
        S = T if pad_rows else len(wants)
        width = max(width, 1, -(-max_ctx // B))
        G = len(cache.groups)
        head = np.empty(3 * T + R + S + G * (T + R * width), np.int32)
        as_i32 = lambda v: np.asarray(v, dtype=np.int32)
        counts, starts, state_slots, want_counts, tokens, wants = map(as_i32, (counts, starts, state_slots, want_counts, tokens, wants))
        # the block tables are read where they lie (one row per request slot), nothing of them passes through Python
        rc_, got = host.step_layout(counts, starts, state_slots, tokens, want_counts, wants, pad_rows,
                                    cache.padding_state_slot, width, B, [g.tables for g in cache.groups], state_slots, head)
        if rc_ == -2:
            raise AssertionError("a row would be written into a page that was given back")
        if rc_ == -3:
            raise AssertionError("the step's description contradicts itself (counts, wanted places or table rows)")
        if rc_ != head.size or (got.T, got.R, got.S, got.width, got.max_context) != (T, R, S, width, max_ctx):
            raise RuntimeError(f"the step layout wrote {rc_} of {head.size} entries")
        parts = [head]
        # what the parts want to know about this batch beyond that: each planner once
        batch = StepBatch(segments, T, R, max_ctx, B, cache, bool(pad_rows))
        plans = []
        for pl in self.planners():
            plan = pl.plan(batch)
            names = sorted(plan.arrays)
            arrays = [np.ascontiguousarray(plan.arrays[n], dtype=np.int32).reshape(-1) for n in names]
            plans.append((pl.key, names, [a.size for a in arrays], plan.facts))
            parts += arrays
        sizes = dict(T=T, R=R, S=S, width=width, plans=plans, max_context=max_ctx)
        return parts, sizes, segments

    def _context(self, dev: torch.Tensor, sizes, segments) -> StepContext:
        """Slices one device buffer (laid out as ``_layout`` says) into the step's tensors."""
        T, R, S, width = sizes["T"], sizes["R"], sizes["S"], sizes["width"]
        o = 0

        def take(n):
            nonlocal o
            v = dev[o:o + n]
            o += n
            return v

        token_ids, positions, row_req, state_slots, selected = take(T), take(T), take(T), take(R), take(S)
        groups = []
        for _ in self.cache.groups:
            slots = take(T)
            table = take(R * width).view(R, width)
            groups.append(GroupStep(table, slots))
        plans = {}
        for key, names, counts, facts in sizes["plans"]:
            plans[key] = StepPlan({n: take(c) for n, c in zip(names, counts)}, dict(facts))
        return StepContext(T, R, token_ids, positions, row_req, state_slots, selected, S, groups, segments,
                           sizes["max_context"], plans)

    def _describe(self, entries: Sequence[StepEntry]) -> StepContext:
        parts, sizes, segments = self._layout(entries)
        dev = torch.from_numpy(np.concatenate(parts)).to(self.device, non_blocking=False)
        return self._context(dev, sizes, segments)

    def step(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs the entries' tokens as one batch from the cache and returns fp32 logits
        [sum(len(want)), vocab] in the order of the entries and of their ``want``.

        ``feed``: an int32 tensor on the device with one token per entry (every entry then brings one placeholder
        token): the token ids are taken from it on the device, so a step can be launched before the host has read
        the tokens that the step before it sampled."""
        if feed is not None and (any(len(e.tokens) != 1 for e in entries) or feed.numel() < len(entries)):
            raise StepError("tokens fed on the device stand for one token of every entry")
        fresh = [e.rid for e in entries if not self.cache.has(e.rid)]
        self.prepare_cache(entries)
        try:
            if self.graphs is not None and self.graphs.takes(entries):
                logits = self.graphs.run(entries, feed)
            else:
                ctx = self._describe(entries)
                if feed is not None:
                    ctx.token_ids[:len(entries)].copy_(feed[:len(entries)])
                logits = self.model.forward(ctx, self.cache.slots)
        except BaseException:
            # the step did not run to its end: the pages begun for it go back and the requests it opened close, so
            # that the cache is as it was before the step (what the kernels may have stored lies beyond every length)
            for e in entries:
                if e.rid in fresh:
                    self.cache.close(e.rid)
                else:
                    self.cache.rollback_write(e.rid)
            raise
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        self.steps += 1
        self.rows += sum(len(e.tokens) for e in entries)
        return logits

    def finish(self, rid) -> None:
        """The request is done (or preempted): its pages and state slot go back."""
        if self.cache.has(rid):
            self.cache.close(rid)
