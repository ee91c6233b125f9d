"""Generation: requests in, token ids out, through the scheduler and the step function.

The reference's loop for one request (engine/Engine.java:502-788): prefill in chunks with logits only for
the last one, then sample -> stop check -> emit -> feed the token; finish reasons "stop" (a token of the
eos set, which is not emitted, :696-699), "length" (min(max_tokens, ctx - prompt), :619, :824) and
"cancelled". The reference runs one thread per request and merges their calls into passes
(engine/BatchGroup.java:353-433); here one loop owns all requests (the design the reference weighed and
left, docs/25-scheduler.md:255-261).

Lookahead (the reference pipelines the greedy steps of a lone slot on the device, model/Backend.java:346-369):
when a pass holds nothing but the single tokens of every running request, and their samplers neither punish nor
report, the sampled tokens stay on the device. The next pass, if it is the same requests again, is launched with
its token ids taken from there, and only then does the host read the tokens of the pass before, finish who
reached a stop token and publish pages, while the GPU is already busy. A request that stops on a token has then
run one row too many, which is dropped with its cache. Anything else (an arrival, a cancellation, a request at
its limit, pages running short) reads the tokens first and goes the plain way.
"""
from __future__ import annotations

import dataclasses

import time
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence

from ..sampling import SamplerState, SamplingParams, sample_rows, select_rows
from .scheduler import FINISHED, RUNNING, Request, Scheduler, SchedulerConfig
from .step import StepEntry


@dataclass(frozen=True)
class TokenLogprob:
    """engine/TokenLogprob.java:14: a generated token's natural-log probability under the raw logits (before
    penalties, bias, temperature or truncation), and the most likely tokens at that position with theirs."""
    token: int
    logprob: float
    top_tokens: tuple = ()
    top_logprobs: tuple = ()


@dataclass
class GenerationResult:
    rid: Any
    tokens: List[int]
    finish_reason: str
    stats: Dict[str, float] = field(default_factory=dict)
    logprobs: Optional[List[TokenLogprob]] = None  # one per generated token when SamplingParams.logprobs
    # one per prompt token when SamplingParams.prompt_logprobs; the first is None: nothing predicts it (Engine.java:61-62)
    prompt_logprobs: Optional[List[Optional[TokenLogprob]]] = None

    def cumulative_logprob(self) -> float:
        """The sequence's log-likelihood (engine/Engine.java:70-77); needs logprobs."""
        if self.logprobs is None:
            raise ValueError("the request did not ask for logprobs")
        return float(sum(lp.logprob for lp in self.logprobs))


class Engine:
    def __init__(self, runner, config: Optional[SchedulerConfig] = None, eos_token_ids: Sequence[int] = (),
                 sample_fn: Callable = sample_rows, clock: Callable[[], float] = time.monotonic,
                 select_fn: Optional[Callable] = None, lookahead: bool = True):
        self.runner = runner
        if config is None:
            config = SchedulerConfig(max_positions=runner.max_positions)
        elif config.max_positions > runner.max_positions:
            # one limit: the scheduler never plans a position the runner (and the model's tables) was not built for
            config = dataclasses.replace(config, max_positions=runner.max_positions)
        self.config = config
        self.scheduler = Scheduler(self.config, runner.cache, clock)
        self.eos = set(eos_token_ids)
        self.sample_fn = sample_fn
        self.requests: Dict[Any, Request] = {}
        self._next_id = 0
        self.on_token: Optional[Callable[[Any, int], None]] = None
        # the selection alone, its result left on the device; with another sample_fn and none given there is no lookahead
        self.select_fn = select_fn if select_fn is not None else (select_rows if sample_fn is sample_rows else None)
        self.lookahead = lookahead and self.select_fn is not None
        self._unread: Optional[tuple] = None  # (requests, their sampled tokens on the device) of the pass not read yet
        self.lookahead_passes = 0
        self._host_tokens: list = []  # two pinned buffers for sampled tokens that take turns
        self._host_turn = 0

    # ------------------------------------------------------------------------------------------ requests

    PRIORITIES = {"interactive": 0, "background": 1}  # engine/Priority.java

    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None, rid=None, priority=0,
                    session: Optional[str] = None):
        """``priority``: "interactive" (0, the default) or "background" (1): background work gives way to
        interactive requests and is aged so that it is not starved (the scheduler's classes). ``session``: requests
        of one session share the limit ``SchedulerConfig.session_max_running`` on how many of them run at once."""
        params = params or SamplingParams()
        priority = self.PRIORITIES.get(priority, priority)
        if rid is None:
            rid = self._next_id
            self._next_id += 1
        if rid in self.requests and self.requests[rid].status != FINISHED:
            raise ValueError(f"request id {rid!r} is in use")
        vocab = self.runner.vocab
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"prompt token {t} is outside the vocabulary of {vocab}")
        r = self.scheduler.add(rid, [int(t) for t in prompt], params, SamplerState(params, vocab, prompt), priority, session)
        r.stats = {"arrival": time.perf_counter(), "prompt_tokens": len(r.prompt)}
        self.requests[rid] = r
        return rid

    def cancel(self, rid) -> None:
        """The request ends with "cancelled" at the next step boundary (engine/Engine.java:565-575, :649-667)."""
        if rid in self.requests:
            self.requests[rid].cancelled = True

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work() or self._unread is not None

    # ------------------------------------------------------------------------------------------ stepping

    def step(self) -> List[Request]:
        """One pass: plan, run, sample, finish. Returns the requests that finished in it."""
        sch = self.scheduler
        done: List[Request] = []
        if self._unread is not None:
            if self._same_again():
                return self._step_ahead()
            done += self._read_tokens()
        for r in list(sch.running) + list(sch.waiting):
            if r.cancelled:
                sch.finish(r, "cancelled")
                done.append(self._close(r))
        for r in list(sch.running) + list(sch.waiting):
            if r.status != FINISHED and sch.limit(r) <= len(r.output):
                sch.finish(r, "length")
                done.append(self._close(r))
        before = {id(r) for r in sch.running} | {id(r) for r in sch.waiting}
        picks = sch.plan()
        for r in self.requests.values():  # a lone request the pool cannot hold was finished by the planner
            if r.status == FINISHED and id(r) in before and "end" not in r.stats:
                done.append(self._close(r))
        if not picks:
            return done
        entries = []
        echo = []  # (request, rows of the logits that predict prompt tokens, those tokens)
        n_rows = 0
        sample_rows = []
        for p in picks:
            r = p.request
            toks = r.tokens[r.computed:r.computed + p.n]
            want = []
            if r.params.prompt_logprobs and len(r.prompt_logprobs) < len(r.prompt):
                # the row at position q predicts prompt token q + 1 (Engine.java:896-908: every row's logits)
                if not r.prompt_logprobs:
                    r.prompt_logprobs.append(None)
                first = max(r.computed, len(r.prompt_logprobs) - 1)  # after a preemption: what is not reported yet
                last = min(r.computed + p.n, len(r.prompt) - 1)
                want = [q - r.computed for q in range(first, last)]
                if want:
                    echo.append((r, list(range(n_rows, n_rows + len(want))), r.prompt[first + 1:last + 1]))
            if p.wants_logits:
                sample_rows.append(n_rows + len(want))
                want.append(p.n - 1)
            n_rows += len(want)
            entries.append(StepEntry(r.rid, toks, want))
            if "first_scheduled" not in r.stats:
                r.stats["first_scheduled"] = time.perf_counter()
        logits = self.runner.step(entries)
        wanting = [p.request for p in picks if p.wants_logits]
        sch.computed(picks)
        if echo:
            self._prompt_logprobs(logits, echo)
            logits = logits[sample_rows] if sample_rows else logits[:0]
        if wanting and self._may_defer(picks):
            self._unread = self._leave_on_device(wanting, self.select_fn(logits, [r.sampler for r in wanting]))
            for r in wanting:
                r.unread = 1
            return done
        if wanting:
            lp_rows = [i for i, r in enumerate(wanting) if r.params.logprobs]
            raw = logits[lp_rows].clone() if lp_rows else None  # sampling may change the logits in place
            tokens = self.sample_fn(logits, [r.sampler for r in wanting])
            reports = self._logprobs(raw, [wanting[i] for i in lp_rows], [int(tokens[i]) for i in lp_rows]) if lp_rows else {}
            now = time.perf_counter()
            for r, tok in zip(wanting, tokens):
                tok = int(tok)
                if "first_token" not in r.stats:
                    r.stats["first_token"] = now
                if tok in self.eos and not r.params.ignore_eos:
                    sch.finish(r, "stop")  # the eos token is not emitted
                    done.append(self._close(r))
                    continue
                r.output.append(tok)
                if id(r) in reports:
                    r.logprobs.append(reports[id(r)])
                r.sampler.accept(tok)
                if self.on_token:
                    self.on_token(r.rid, tok)
                if len(r.output) >= sch.limit(r):
                    sch.finish(r, "length")
                    done.append(self._close(r))
        return done

    # ------------------------------------------------------------------------------------------ lookahead

    def _may_defer(self, picks) -> bool:
        """The pass was nothing but one token of every running request, nobody waits, and no sampler needs the
        tokens on the host (penalties, bias, reports): the tokens may stay on the device for now."""
        sch = self.scheduler
        if not self.lookahead or sch.waiting or len(picks) != len(sch.running):
            return False
        for p in picks:
            r = p.request
            if p.n != 1 or not p.wants_logits or r.computed < len(r.prompt) or not r.params.plain \
                    or r.params.logprobs or r.params.prompt_logprobs:
                return False
        return True

    def _same_again(self) -> bool:
        """The next pass would be the same requests with the tokens not read yet: nothing arrived, nobody was
        cancelled or is at its limit, and the pages are there."""
        sch = self.scheduler
        reqs = self._unread[0]
        if sch.waiting or len(reqs) != len(sch.running) or len(reqs) > self.config.max_batch_tokens:
            return False
        if any(a is not b for a, b in zip(reqs, sch.running)):
            return False
        for r in reqs:
            if r.cancelled or r.status != RUNNING or len(r.output) + r.unread >= sch.limit(r):
                return False
        free = list(self.runner.cache.free_pages())
        for r in reqs:
            for gi, need in enumerate(self.runner.cache.pages_needed(r.rid, 1)):
                free[gi] -= need
        return all(f >= 0 for f in free)

    def _step_ahead(self) -> List[Request]:
        """Launches the next pass with its tokens taken from the device, then reads the tokens of the one before."""
        sch = self.scheduler
        reqs, tokens_dev = self._unread[:2]
        entries = [StepEntry(r.rid, [0], [0]) for r in reqs]
        logits = self.runner.step(entries, feed=tokens_dev)
        sch.count_pass([(1, r.computed) for r in reqs])
        for r in reqs:
            r.computed += 1
            r.last_pass = sch.passes - 1
        self.lookahead_passes += 1
        ahead = self._leave_on_device(reqs, self.select_fn(logits, [r.sampler for r in reqs]))[1:]
        done = self._read_tokens()
        alive = [r for r in reqs if r.status == RUNNING]
        if len(alive) == len(reqs):
            self._unread = (reqs,) + ahead
            for r in reqs:
                r.unread = 1
            return done
        # somebody stopped on the token just read: its row in the pass just launched is dropped with its cache; the
        # others' tokens are read at once, so that the books are plain again
        self._unread = (reqs,) + ahead
        for r in alive:
            r.unread = 1
        return done + self._read_tokens()

    def _leave_on_device(self, reqs, tokens_dev) -> tuple:
        """The sampled tokens stay on the device for the next pass to take; their copy into pinned host memory is put
        into the stream at once, right behind the kernel that made them and before the next pass is launched, with
        an event behind it: waiting for that event waits for these tokens only. (Read later, the copy would stand
        behind the pass launched meanwhile: the host would wait for that whole pass and the GPU would idle while the
        host prepares the next one.)"""
        import torch
        if not isinstance(tokens_dev, torch.Tensor) or not tokens_dev.is_cuda or tokens_dev.dtype != torch.int32:
            return reqs, tokens_dev, None, None
        from ..kernels import ops
        n = tokens_dev.numel()
        if len(self._host_tokens) < 2 or self._host_tokens[0].numel() < n:
            if self._host_tokens:
                # copy kernels that write the old pinned blocks may still be queued; the host allocator that gets the
                # blocks back knows nothing of kernels, so the stream is drained first (the batch grew: rare)
                torch.cuda.current_stream().synchronize()
            size = max(64, 1 << (n - 1).bit_length())
            self._host_tokens = [torch.empty(size, dtype=torch.int32).pin_memory() for _ in range(2)]
        self._host_turn ^= 1
        host = self._host_tokens[self._host_turn][:n]
        ops.copy_words(tokens_dev.contiguous(), host)
        arrived = torch.cuda.Event()
        arrived.record()
        return reqs, tokens_dev, host, arrived

    def _read_tokens(self) -> List[Request]:
        """Brings the tokens that stayed on the device to the host and does what follows a sampled token."""
        sch = self.scheduler
        reqs, tokens_dev, host, arrived = self._unread
        self._unread = None
        if arrived is not None:
            arrived.synchronize()
            tokens = host.tolist()
        else:
            tokens = tokens_dev.tolist()
        now = time.perf_counter()
        done: List[Request] = []
        cache = self.runner.cache
        for r, tok in zip(reqs, tokens):
            if r.status != RUNNING or not r.unread:
                continue  # finished meanwhile: the row is dropped
            r.unread = 0
            tok = int(tok)
            if "first_token" not in r.stats:
                r.stats["first_token"] = now
            if tok in self.eos and not r.params.ignore_eos:
                sch.finish(r, "stop")
                done.append(self._close(r))
                continue
            r.output.append(tok)
            r.sampler.accept(tok)
            if self.on_token:
                self.on_token(r.rid, tok)
            if cache.sharing and cache.has(r.rid) and r.computed // cache.page_size > cache.published_pages(r.rid):
                cache.publish(r.rid, r.tokens[:r.computed])
            if len(r.output) >= sch.limit(r):
                sch.finish(r, "length")
                done.append(self._close(r))
        return done

    @staticmethod
    def _logprobs(raw, requests, tokens) -> dict:
        """request -> TokenLogprob of the token just chosen for it, from the raw logits rows."""
        import torch
        from ..kernels import ops
        top = max(r.params.top_logprobs for r in requests)
        lp, ids, tlp = ops.token_logprobs(raw, torch.tensor(tokens, dtype=torch.int32, device=raw.device), top)
        lp, ids, tlp = lp.tolist(), ids.tolist(), tlp.tolist()
        out = {}
        for i, r in enumerate(requests):
            k = r.params.top_logprobs
            out[id(r)] = TokenLogprob(tokens[i], lp[i], tuple(ids[i][:k]), tuple(tlp[i][:k]))
        return out

    @staticmethod
    def _prompt_logprobs(logits, echo) -> None:
        import torch
        from ..kernels import ops
        rows = [i for _, idx, _ in echo for i in idx]
        tokens = [t for _, _, toks in echo for t in toks]
        top = max(r.params.top_logprobs for r, _, _ in echo)
        dev = logits.device
        lp, ids, tlp = ops.token_logprobs(logits[torch.tensor(rows, device=dev)],
                                          torch.tensor(tokens, dtype=torch.int32, device=dev), top)
        lp, ids, tlp = lp.tolist(), ids.tolist(), tlp.tolist()
        i = 0
        for r, idx, toks in echo:
            k = r.params.top_logprobs
            for t in toks:
                r.prompt_logprobs.append(TokenLogprob(t, lp[i], tuple(ids[i][:k]), tuple(tlp[i][:k])))
                i += 1

    def _close(self, r: Request) -> Request:
        r.stats["end"] = time.perf_counter()
        s = r.stats
        s["generated_tokens"] = len(r.output)
        if "first_token" in s:
            s["prefill_ms"] = (s["first_token"] - s.get("first_scheduled", s["arrival"])) * 1e3
            s["decode_ms"] = (s["end"] - s["first_token"]) * 1e3
            s["tok_per_sec"] = (len(r.output) - 1) / max(1e-9, s["end"] - s["first_token"]) if len(r.output) > 1 else 0.0
        s["preemptions"] = r.preemptions
        s["cached_tokens"] = r.cached_tokens
        return r

    # ------------------------------------------------------------------------------------------ whole runs

    def generate(self, prompts: Sequence[Sequence[int]], params=None) -> List[GenerationResult]:
        """Runs the prompts to the end (params: one SamplingParams for all, or one per prompt); results in the
        order of the prompts. The reference's Engine.generate returns (text, tokens, finish reason, stats) for
        one prompt (engine/Engine.java:368-376); this engine has no tokenizer, so tokens only."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_unfinished():
            self._progress()
        return [self._result(rid) for rid in rids]

    def generate_choices(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                         n: int = 1) -> List[GenerationResult]:
        """n independent completions of one prompt (engine/Engine.java:378-447): choice i of a seeded request
        samples with seed + i, choice 0 exactly like a single request; an unseeded one draws a fresh seed per
        choice. The reference runs the choices one after the other and takes the prompt from its prefix cache;
        here choice 0 computes the prompt, then the others are admitted, take its pages over when the cache
        shares prefixes (else each computes the prompt), and all decode together."""
        if n < 1:
            raise ValueError(f"n must be at least 1, got {n}")
        params = params or SamplingParams()
        rids = [self.add_request(prompt, params)]
        first = self.requests[rids[0]]
        while first.status != FINISHED and first.computed < len(first.prompt):
            self._progress()
        from dataclasses import replace
        later = replace(params, prompt_logprobs=False)  # the prompt is the same for every choice (Engine.java:431-441)
        for i in range(1, n):
            rids.append(self.add_request(prompt, later.with_seed(params.seed + i) if params.seed >= 0 else later))
        while any(self.requests[rid].status != FINISHED for rid in rids):
            self._progress()
        results = [self._result(rid) for rid in rids]
        for r in results[1:]:
            r.prompt_logprobs = results[0].prompt_logprobs
        return results

    def _progress(self) -> None:
        before = self.runner.steps
        finished = self.step()
        if self.runner.steps == before and not finished and self.has_unfinished():
            raise RuntimeError("the scheduler made no progress: " + str(self.stats()))

    def _result(self, rid) -> GenerationResult:
        r = self.requests.pop(rid)
        return GenerationResult(rid, list(r.output), r.finish_reason, dict(r.stats),
                                list(r.logprobs) if r.params.logprobs else None,
                                list(r.prompt_logprobs) if r.params.prompt_logprobs else None)

    def stats(self) -> dict:
        return {"scheduler": self.scheduler.stats(), "cache": self.runner.cache.stats(),
                "steps": self.runner.steps, "rows": self.runner.rows}
