"""The scheduler's decisions and the engine loop, on the host with a fake model and the real cache manager."""
import random

import pytest

from fakes import FakeRunner, argmax_sampler, expected_generation
from jllm_serve_amd.engine import Engine, SchedulerConfig
from jllm_serve_amd.sampling import SamplingParams


def make(pool_tokens=64, page_size=4, max_requests=4, window=0, prefix_share=False, read_pages=False, **cfg):
    cfg.setdefault("max_positions", 256)
    runner = FakeRunner(page_size=page_size, pool_tokens=pool_tokens, max_requests=max_requests, window=window,
                        prefix_share=prefix_share, read_pages=read_pages, max_positions=cfg["max_positions"])
    eng = Engine(runner, SchedulerConfig(**cfg), sample_fn=argmax_sampler)
    orig_close = runner.cache.close

    def close(rid):  # the fake model forgets a request when its cache goes (finish or preemption)
        orig_close(rid)
        runner.model.history.pop(rid, None)
    runner.cache.close = close
    return eng, runner


def greedy(n):
    return SamplingParams.greedy_params(max_tokens=n)


def test_engine_call_pattern():
    """A prompt [5, 6, 7, 8] + 2 tokens: one call (0, 4), then (4, 1); the last sampled token is never fed
    (the recording-backend check of T/SmokeTest.java:1458-1475)."""
    eng, runner = make(max_batch_tokens=64, prefill_chunk=64)
    res = eng.generate([[5, 6, 7, 8]], greedy(2))[0]
    assert runner.model.calls == [[(0, 0, 4)], [(0, 4, 1)]]
    exp, why = expected_generation([5, 6, 7, 8], 2, 97)
    assert res.tokens == exp and res.finish_reason == "length"
    runner.cache.check()
    assert runner.cache.stats()["groups"][0]["used"] == 0


def test_chunked_prefill_and_budget():
    eng, runner = make(pool_tokens=256, max_batch_tokens=20, prefill_chunk=16, min_chunk=4)
    prompts = [list(range(1, 41)), list(range(3, 12)), [9]]
    res = eng.generate(prompts, greedy(6))
    for p, r in zip(prompts, res):
        assert r.tokens == expected_generation(p, 6, 97)[0]
    for call in runner.model.calls:
        assert sum(n for _, _, n in call) <= 20
        for _, _, n in call:
            assert n <= 16
    assert any(len(c) > 1 for c in runner.model.calls), "portions and decode rows should share passes"
    # portions come first in a pass, single decode rows after them (PassPlanner.java:70-73)
    for call in runner.model.calls:
        kinds = [n > 1 for _, _, n in call]
        assert kinds == sorted(kinds, reverse=True) or all(n == 1 for _, _, n in call)


def test_min_chunk_waits_for_room():
    """PassPlanner.java:95-99: a portion is trimmed to the leftover only if that is at least min_chunk rows."""
    eng, runner = make(pool_tokens=256, max_batch_tokens=20, prefill_chunk=64, min_chunk=16, max_requests=8)
    for i in range(6):
        eng.add_request([i + 1], greedy(40))
    for _ in range(3):
        eng.step()  # six requests decode: 6 rows a pass
    eng.add_request(list(range(1, 31)), greedy(2))
    eng.step()
    last = runner.model.calls[-1]
    assert [n for _, _, n in last if n > 1] == [], "14 rows of room < min_chunk 16: the prompt waits"
    for r in list(eng.scheduler.running)[:2]:
        eng.cancel(r.rid)
    eng.step()
    last = runner.model.calls[-1]
    assert [n for _, _, n in last if n > 1] == [16], "with 4 riders the leftover of 16 rows is taken"


def test_oldest_goes_alone_when_nothing_fits():
    """PassPlanner.java:105-110: a 30-row item with budget 10 still goes, trimmed to the budget."""
    eng, runner = make(pool_tokens=256, max_batch_tokens=10, prefill_chunk=64, min_chunk=16)
    res = eng.generate([list(range(1, 31))], greedy(1))[0]
    assert [c[0][2] for c in runner.model.calls] == [10, 10, 10]
    assert res.tokens == expected_generation(list(range(1, 31)), 1, 97)[0]


def test_eos_stops_and_is_not_emitted():
    prompt = [4, 8, 15]
    free_run, _ = expected_generation(prompt, 10, 97)
    eos = free_run[3]
    runner = FakeRunner()
    eng = Engine(runner, SchedulerConfig(max_positions=256), eos_token_ids=[eos], sample_fn=argmax_sampler)
    r = eng.generate([prompt], greedy(10))[0]
    assert r.finish_reason == "stop" and r.tokens == free_run[:free_run.index(eos)]
    r2 = eng.generate([prompt], SamplingParams.greedy_params(max_tokens=10, ignore_eos=True))[0]
    assert r2.finish_reason == "length" and r2.tokens == free_run


def test_context_limit_and_prompt_too_long():
    eng, _ = make(pool_tokens=256, max_positions=12)
    r = eng.generate([[1, 2, 3, 4, 5]], greedy(100))[0]
    assert r.finish_reason == "length" and len(r.tokens) == 12 - 5  # min(max_tokens, ctx - prompt), Engine.java:619
    with pytest.raises(ValueError):
        eng.add_request(list(range(12)), greedy(1))  # prompt >= ctx, Engine.java:505-507
    with pytest.raises(ValueError):
        eng.add_request([], greedy(1))
    with pytest.raises(ValueError):
        eng.add_request([97], greedy(1))


def test_prompt_that_can_never_fit_is_refused_at_submit():
    eng, _ = make(pool_tokens=16)
    with pytest.raises(ValueError, match="never fit"):
        eng.add_request(list(range(1, 17)), greedy(1))


def test_out_of_pages_preempts_newest_and_recomputes():
    """Pool of 12 pages x 4: three requests growing to 28 tokens each cannot all stay. The newest running one
    is preempted, its pages return, it is computed again later; every answer equals the unpreempted one."""
    eng, runner = make(pool_tokens=48, page_size=4, max_batch_tokens=64, prefill_chunk=64, min_chunk=1)
    prompts = [[1, 2, 3, 4, 5, 6, 7, 8], [11, 12, 13, 14, 15, 16, 17, 18], [21, 22, 23, 24, 25, 26, 27, 28]]
    res = eng.generate(prompts, greedy(20))
    for p, r in zip(prompts, res):
        assert r.tokens == expected_generation(p, 20, 97)[0] and r.finish_reason == "length"
    assert eng.scheduler.preemptions > 0
    assert max(r.stats["preemptions"] for r in res) > 0 and res[0].stats["preemptions"] == 0, "the oldest is never the victim"
    runner.cache.check()
    assert all(g["used"] == 0 for g in runner.cache.stats()["groups"])


def test_lone_request_that_outgrows_the_pool_ends_with_length():
    eng, runner = make(pool_tokens=16, page_size=4)
    r = eng.generate([[1, 2, 3]], greedy(100))[0]
    assert r.finish_reason == "length"
    assert r.tokens == expected_generation([1, 2, 3], len(r.tokens), 97)[0]
    assert 12 <= len(r.tokens) + 3 <= 17
    runner.cache.check()


def test_no_admission_without_pages():
    eng, runner = make(pool_tokens=32, page_size=4, max_batch_tokens=64, prefill_chunk=64)
    a = eng.add_request(list(range(1, 25)), greedy(4))   # 6 of 8 pages
    b = eng.add_request(list(range(30, 50)), greedy(4))  # needs 5: must wait
    eng.step()
    assert [r.rid for r in eng.scheduler.running] == [a] and [r.rid for r in eng.scheduler.waiting] == [b]
    while eng.has_unfinished():
        eng.step()
    assert eng.scheduler.preemptions == 0
    assert eng.requests[b].output == expected_generation(list(range(30, 50)), 4, 97)[0]


def test_max_running_and_cancel():
    eng, runner = make(pool_tokens=256, max_running=2, max_requests=4)
    ids = [eng.add_request([i + 1, i + 2], greedy(50)) for i in range(3)]
    eng.step()
    assert len(eng.scheduler.running) == 2 and len(eng.scheduler.waiting) == 1
    eng.cancel(ids[0])
    done = eng.step()
    assert [r.rid for r in done] == [ids[0]] and done[0].finish_reason == "cancelled"
    assert len(eng.scheduler.running) == 2  # the waiting one took the slot
    runner.cache.check()


def test_random_workloads_match_free_running():
    rng = random.Random(5)
    for trial in range(15):
        window = rng.choice([0, 0, 6])
        eng, runner = make(pool_tokens=rng.choice([64, 96, 160]), page_size=rng.choice([2, 4, 8]),
                           max_batch_tokens=rng.choice([8, 24, 64]), prefill_chunk=rng.choice([4, 16, 64]),
                           min_chunk=rng.choice([1, 4, 16]), max_requests=rng.choice([2, 4]), window=window)
        prompts = [[rng.randrange(97) for _ in range(rng.randrange(1, 40))] for _ in range(rng.randrange(1, 7))]
        params = [greedy(rng.randrange(1, 25)) for _ in prompts]
        pending = list(zip(prompts, params))
        rids = {}
        while pending or eng.has_unfinished():
            if pending and rng.random() < 0.5:
                p, sp = pending.pop(0)
                rids[eng.add_request(p, sp)] = (p, sp)
            eng.step()
            runner.cache.check()
        for rid, (p, sp) in rids.items():
            r = eng.requests[rid]
            exp = expected_generation(p, sp.max_tokens, 97)[0]
            if r.stats["preemptions"] == 0 or r.finish_reason == "length":
                assert r.output == exp[:len(r.output)]
            if len(r.output) < sp.max_tokens:
                assert r.finish_reason == "length" and len(eng.scheduler.running) == 0
        assert all(g["used"] == 0 for g in runner.cache.stats()["groups"])


# ------------------------------------------------------------------------------------------ prefix sharing

def test_fake_model_that_reads_pages_matches_the_plain_one():
    eng, runner = make(pool_tokens=48, page_size=4, max_batch_tokens=16, prefill_chunk=8, min_chunk=1, read_pages=True)
    prompts = [[1, 2, 3, 4, 5, 6, 7, 8], [11, 12, 13, 14, 15, 16, 17, 18, 19], [21, 22, 23]]
    for p, r in zip(prompts, eng.generate(prompts, greedy(20))):
        assert r.tokens == expected_generation(p, 20, 97)[0]
    assert eng.scheduler.preemptions > 0, "pages were reused; a stale row would have changed a token"


def test_a_shared_start_is_computed_once():
    eng, runner = make(pool_tokens=256, page_size=4, max_batch_tokens=64, prefill_chunk=64, prefix_share=True)
    stem = list(range(40, 58))  # 18 tokens: four full pages and two rows
    first = eng.generate([stem + [1, 2]], greedy(6))[0]
    assert first.tokens == expected_generation(stem + [1, 2], 6, 97)[0] and first.stats["cached_tokens"] == 0
    calls_before = len(runner.model.calls)
    second = eng.generate([stem + [3]], greedy(6))[0]
    assert second.tokens == expected_generation(stem + [3], 6, 97)[0]
    assert second.stats["cached_tokens"] == 18, "four shared pages and two copied rows"
    assert runner.model.calls[calls_before] == [(1, 18, 1)], "only the token that differs is computed"
    # the very same prompt again: everything but its last token comes from the tree (Engine.java:518-521)
    third = eng.generate([stem + [1, 2]], greedy(6))[0]
    assert third.tokens == first.tokens and third.stats["cached_tokens"] == 19
    # and a continuation of the first answer finds the generated tokens too (published as they were computed)
    turn2 = stem + [1, 2] + first.tokens[:5] + [9]
    fourth = eng.generate([turn2], greedy(3))[0]
    assert fourth.tokens == expected_generation(turn2, 3, 97)[0] and fourth.stats["cached_tokens"] >= 24
    runner.cache.check()
    st = runner.cache.stats()
    assert st["prefix"]["hits"] == 3 and st["groups"][0]["used"] == st["prefix"]["nodes"] == st["prefix"]["idle"]


def test_requests_running_together_share_pages():
    eng, runner = make(pool_tokens=64, page_size=4, max_batch_tokens=64, prefill_chunk=64, prefix_share=True)
    stem = list(range(10, 30))
    eng.generate([stem + [5]], greedy(1))
    rids = [eng.add_request(stem + [i], greedy(8)) for i in (1, 2, 3)]
    eng.step()
    runner.cache.check()
    tables = [runner.cache.table(r, 0) for r in rids]
    assert tables[0][:5] == tables[1][:5] == tables[2][:5], "five full pages held once"
    assert runner.cache.stats()["groups"][0]["used"] == 5 + 3
    while eng.has_unfinished():
        eng.step()
        runner.cache.check()
    for rid, i in zip(rids, (1, 2, 3)):
        assert eng.requests[rid].output == expected_generation(stem + [i], 8, 97)[0]


def test_a_preempted_request_finds_its_pages_again():
    eng, runner = make(pool_tokens=48, page_size=4, max_batch_tokens=64, prefill_chunk=64, min_chunk=1, prefix_share=True)
    prompts = [[1, 2, 3, 4, 5, 6, 7, 8], [11, 12, 13, 14, 15, 16, 17, 18], [21, 22, 23, 24, 25, 26, 27, 28]]
    res = eng.generate(prompts, greedy(20))
    for p, r in zip(prompts, res):
        assert r.tokens == expected_generation(p, 20, 97)[0] and r.finish_reason == "length"
    assert eng.scheduler.preemptions > 0 and runner.cache.stats()["prefix"]["evictions"] > 0
    runner.cache.check()


def test_random_workloads_with_sharing():
    rng = random.Random(9)
    hits = 0
    for trial in range(20):
        eng, runner = make(pool_tokens=rng.choice([64, 96, 160]), page_size=rng.choice([2, 4, 8]),
                           max_batch_tokens=rng.choice([8, 24, 64]), prefill_chunk=rng.choice([4, 16, 64]),
                           min_chunk=rng.choice([1, 4, 16]), max_requests=rng.choice([2, 4]), prefix_share=True)
        stems = [[rng.randrange(97) for _ in range(rng.randrange(4, 30))] for _ in range(2)]
        prompts = [rng.choice(stems)[:rng.randrange(1, 30)] + [rng.randrange(97) for _ in range(rng.randrange(1, 8))]
                   for _ in range(rng.randrange(2, 9))]
        params = [greedy(rng.randrange(1, 25)) for _ in prompts]
        pending = list(zip(prompts, params))
        rids = {}
        while pending or eng.has_unfinished():
            if pending and rng.random() < 0.4:
                p, sp = pending.pop(0)
                rids[eng.add_request(p, sp)] = (p, sp)
            eng.step()
            runner.cache.check()
        for rid, (p, sp) in rids.items():
            r = eng.requests[rid]
            exp = expected_generation(p, sp.max_tokens, 97)[0]
            assert r.output == exp[:len(r.output)], "shared, copied and evicted pages never change an answer"
            if len(r.output) < sp.max_tokens:
                assert r.finish_reason == "length"
        st = runner.cache.stats()
        hits += st["prefix"]["hits"]
        assert st["groups"][0]["used"] == st["prefix"]["nodes"]
    assert hits > 20


def test_choices_of_one_prompt_compute_it_once():
    eng, runner = make(pool_tokens=256, page_size=4, max_batch_tokens=64, prefill_chunk=8, prefix_share=True)
    prompt = list(range(30, 51))  # 21 tokens: three portions of at most 8
    res = eng.generate_choices(prompt, greedy(5), n=3)
    exp = expected_generation(prompt, 5, 97)[0]
    assert [r.tokens for r in res] == [exp] * 3, "greedy choices are equal"
    assert [r.stats["cached_tokens"] for r in res] == [0, 20, 20]
    prefill_calls = [c for call in runner.model.calls for c in call if c[2] > 1]
    assert prefill_calls == [(0, 0, 8), (0, 8, 8), (0, 16, 5)], "the prompt is computed by choice 0 only"
    runner.cache.check()
    with pytest.raises(ValueError):
        eng.generate_choices(prompt, greedy(2), n=0)
    # without sharing every choice computes the prompt; the answers are the same
    eng2, runner2 = make(pool_tokens=256, page_size=4, max_batch_tokens=64, prefill_chunk=8)
    assert [r.tokens for r in eng2.generate_choices(prompt, greedy(5), n=2)] == [exp] * 2


def test_choices_use_consecutive_seeds():
    seen = []

    def sampler(logits, states):
        seen.extend(s.seed for s in states)
        return argmax_sampler(logits, states)
    runner = FakeRunner(pool_tokens=128)
    eng = Engine(runner, SchedulerConfig(max_positions=256), sample_fn=sampler)
    eng.generate_choices([1, 2, 3], SamplingParams(seed=40, max_tokens=1), n=3)
    assert sorted(set(seen)) == [40, 41, 42]
    seen.clear()
    eng.generate_choices([1, 2, 3], SamplingParams(seed=-1, max_tokens=1), n=3)
    assert len(set(seen)) == 3, "an unseeded request draws a fresh seed per choice"


# ------------------------------------------------------------------------------------------ classes

class Clock:
    def __init__(self):
        self.now = 0.0

    def __call__(self):
        return self.now


def make_with_clock(**cfg):
    clock = Clock()
    cfg.setdefault("max_positions", 256)
    runner = FakeRunner(page_size=4, pool_tokens=cfg.pop("pool_tokens", 256), max_requests=cfg.pop("max_requests", 4),
                        prefix_share=cfg.pop("prefix_share", False), read_pages=True, max_positions=cfg["max_positions"])
    return Engine(runner, SchedulerConfig(**cfg), sample_fn=argmax_sampler, clock=clock), runner, clock


def first_calls(runner):
    """Request ids in the order in which their first rows ran."""
    order = []
    for call in runner.model.calls:
        for rid, pos, n in call:
            if rid not in order:
                order.append(rid)
    return order


def test_interactive_requests_are_admitted_before_background_ones_and_waiting_promotes():
    eng, runner, clock = make_with_clock(max_running=1, max_batch_tokens=32, prefill_chunk=32, age_promote_s=10.0)
    b1 = eng.add_request([1, 2, 3], greedy(2), priority="background")
    b2 = eng.add_request([4, 5, 6], greedy(2), priority="background")
    i1 = eng.add_request([7, 8, 9], greedy(2))
    i2 = eng.add_request([10, 11, 12], greedy(2), priority="interactive")
    assert [eng.scheduler.rank(eng.requests[r]) for r in (b1, b2, i1, i2)] == [1, 1, 0, 0]
    while eng.has_unfinished():
        eng.step()
    assert first_calls(runner) == [i1, i2, b1, b2], "class first, then arrival (Admission.java:192-214)"
    for rid, p in ((b1, [1, 2, 3]), (i2, [10, 11, 12])):
        assert eng.requests[rid].output == expected_generation(p, 2, 97)[0]
    # a background request that has waited age_promote_s counts as interactive and keeps its place by arrival
    eng, runner, clock = make_with_clock(max_running=1, max_batch_tokens=32, prefill_chunk=32, age_promote_s=10.0)
    b = eng.add_request([1, 2, 3], greedy(2), priority="background")
    clock.now = 9.0
    late = eng.add_request([4, 5, 6], greedy(2), priority="background")
    clock.now = 10.5
    i = eng.add_request([7, 8, 9], greedy(2))
    assert [eng.scheduler.rank(eng.requests[r]) for r in (b, late, i)] == [0, 1, 0]
    while eng.has_unfinished():
        eng.step()
    assert first_calls(runner) == [b, i, late]
    with pytest.raises(ValueError, match="priority"):
        eng.add_request([1], greedy(1), priority=3)


def test_an_interactive_arrival_displaces_the_background_request_that_started_last():
    eng, runner, clock = make_with_clock(max_running=2, max_batch_tokens=32, prefill_chunk=32, prefix_share=True)
    b1 = eng.add_request(list(range(1, 10)), greedy(12), priority="background")
    b2 = eng.add_request(list(range(11, 20)), greedy(12), priority="background")
    for _ in range(4):
        eng.step()
    assert len(eng.scheduler.running) == 2
    i = eng.add_request(list(range(21, 30)), greedy(4))
    eng.step()
    running = [r.rid for r in eng.scheduler.running]
    assert running == [b1, i] and eng.scheduler.displaced == 1 and eng.requests[b2].preemptions == 1
    while eng.has_unfinished():
        eng.step()
        runner.cache.check()
    for rid, p, n in ((b1, range(1, 10), 12), (b2, range(11, 20), 12), (i, range(21, 30), 4)):
        assert eng.requests[rid].output == expected_generation(list(p), n, 97)[0]
    assert eng.requests[b2].cached_tokens >= 8, "the displaced request finds its pages again"
    # engine.preempt = false: the interactive request waits for a place
    eng, runner, clock = make_with_clock(max_running=1, max_batch_tokens=32, prefill_chunk=32, preempt=False)
    b = eng.add_request([1, 2, 3], greedy(5), priority="background")
    eng.step()
    i = eng.add_request([4, 5, 6], greedy(2))
    eng.step()
    assert [r.rid for r in eng.scheduler.running] == [b] and eng.scheduler.displaced == 0


def test_a_background_portion_is_capped_beside_an_interactive_rider():
    eng, runner, clock = make_with_clock(max_batch_tokens=64, prefill_chunk=64, background_chunk_cap=8, min_chunk=4)
    i = eng.add_request([1, 2, 3], greedy(10))
    eng.step()
    long_prompt = [t % 97 for t in range(10, 130)]
    b = eng.add_request(long_prompt, greedy(2), priority="background")
    eng.step()
    assert runner.model.calls[-1] == [(b, 0, 8), (i, 3, 1)], "PassPlanner.java:94-96"
    while eng.requests[i].status != "finished":
        eng.step()
    eng.step()
    assert runner.model.calls[-1][0][2] > 8, "no interactive rider, no cap"
    while eng.has_unfinished():
        eng.step()
    assert eng.requests[b].output == expected_generation(long_prompt, 2, 97)[0]


def test_out_of_pages_takes_a_background_request_first():
    eng, runner, clock = make_with_clock(pool_tokens=40, max_batch_tokens=64, prefill_chunk=64, min_chunk=1)
    b = eng.add_request(list(range(1, 9)), greedy(20), priority="background")
    i1 = eng.add_request(list(range(11, 19)), greedy(20))
    i2 = eng.add_request(list(range(21, 29)), greedy(20))
    while eng.has_unfinished():
        eng.step()
        runner.cache.check()
    assert eng.requests[b].preemptions > 0 and eng.requests[i1].preemptions == 0
    for rid, p in ((b, range(1, 9)), (i1, range(11, 19)), (i2, range(21, 29))):
        assert eng.requests[rid].output == expected_generation(list(p), 20, 97)[0]


def picks_of(eng):
    """The next pass as the reference's tests print it: 'id:rows' in the order of the batch (portions, then riders)."""
    runner = eng.runner
    before = len(runner.model.calls)
    eng.step()
    return " ".join(f"{rid}:{n}" for rid, pos, n in runner.model.calls[before])


def test_planner_vectors_of_the_reference():
    """The worked example of the reference's planner (T/SchedulerPolicyTest.java:60-108), without its verification
    runs (no speculation here): a 256-row chunk beside six decoding requests under budgets 288, 100 and 20; an
    interactive chunk before an older background one until two aging periods have passed; the background cap."""
    def six_riders_and_two_prompts(budget):
        eng, runner, clock = make_with_clock(pool_tokens=4096, max_requests=8, max_batch_tokens=budget, prefill_chunk=256,
                                             min_chunk=16, max_positions=1024)
        for i in range(1, 7):
            eng.add_request([i], greedy(50), rid=f"D{i}")
        eng.step()  # the six one-token prompts; from now on they decode
        eng.add_request([t % 97 for t in range(256)], greedy(4), rid="P-A")
        eng.add_request([t % 89 for t in range(256)], greedy(4), rid="P-B")
        return eng
    # one difference kept on purpose: what the older chunk leaves goes to the next one (26 rows >= min_chunk)
    assert picks_of(six_riders_and_two_prompts(288)) == "P-A:256 P-B:26 D1:1 D2:1 D3:1 D4:1 D5:1 D6:1"
    assert picks_of(six_riders_and_two_prompts(100)) == "P-A:94 D1:1 D2:1 D3:1 D4:1 D5:1 D6:1", "the chunk is trimmed, never the riders"
    assert picks_of(six_riders_and_two_prompts(20)) == "D1:1 D2:1 D3:1 D4:1 D5:1 D6:1", "leftover 14 rows < min_chunk 16: the chunk waits"

    def two_chunks(now_ms):
        eng, runner, clock = make_with_clock(pool_tokens=1024, max_running=1, max_batch_tokens=300, prefill_chunk=300,
                                             min_chunk=16, age_promote_s=0.010)
        clock.now = 0.001
        eng.add_request(list(range(64)), greedy(1), rid="bg", priority="background")
        clock.now = 0.005
        eng.add_request(list(range(1, 65)), greedy(1), rid="ia")
        clock.now = now_ms / 1e3
        return eng
    assert picks_of(two_chunks(6)) == "ia:64", "an interactive chunk goes before an older background one"
    assert picks_of(two_chunks(25)) == "bg:64", "after two aging periods the background chunk counts as interactive and is older"

    eng, runner, clock = make_with_clock(pool_tokens=1024, max_batch_tokens=288, prefill_chunk=256, min_chunk=16,
                                         background_chunk_cap=64, max_positions=512)
    eng.add_request([3], greedy(9), rid="d")
    eng.step()
    eng.add_request([t % 97 for t in range(256)], greedy(1), rid="bg", priority="background")
    assert picks_of(eng) == "bg:64 d:1", "a background chunk riding with an interactive token is capped"
    eng, runner, clock = make_with_clock(pool_tokens=1024, max_batch_tokens=288, prefill_chunk=256, min_chunk=16,
                                         background_chunk_cap=64, max_positions=512)
    eng.add_request([t % 97 for t in range(256)], greedy(1), rid="bg", priority="background")
    assert picks_of(eng) == "bg:256", "alone it is not"
    eng, runner, clock = make_with_clock(pool_tokens=1024, max_batch_tokens=10, prefill_chunk=256, min_chunk=16)
    eng.add_request(list(range(30)), greedy(1), rid="v")
    assert picks_of(eng) == "v:10", "an item larger than the budget still goes, alone, trimmed to the budget"


def test_a_waiting_request_whose_start_is_cached_goes_first_until_the_other_has_waited_long_enough():
    """Among waiting requests of one class the score decides: cached tokens + 2000 per second waited
    (T/SchedulerPolicyTest.java:176-190: the one with 4000 cached tokens gets the freed place first)."""
    def setup():
        eng, runner, clock = make_with_clock(pool_tokens=1024, max_running=1, max_batch_tokens=256, prefill_chunk=256,
                                             prefix_share=True)
        stem = [t % 97 for t in range(3, 103)]
        eng.generate([stem + [1]], greedy(1))  # leaves 100 tokens of the stem in the tree
        busy = eng.add_request([5, 6, 7], greedy(30), rid="busy")
        eng.step()
        return eng, runner, clock, stem
    eng, runner, clock, stem = setup()
    eng.add_request([9] * 20, greedy(1), rid="cold")
    eng.add_request(stem + [2], greedy(1), rid="warm")
    eng.cancel("busy")
    assert picks_of(eng) == "warm:1", "100 cached tokens beat an earlier arrival"
    eng, runner, clock, stem = setup()
    eng.add_request([9] * 20, greedy(1), rid="cold")
    clock.now += 0.06  # 2000 tokens per second: 60 ms are worth 120 tokens
    eng.add_request(stem + [2], greedy(1), rid="warm")
    eng.cancel("busy")
    assert picks_of(eng) == "cold:20"


def test_requests_that_arrive_together_and_start_alike_compute_the_start_once():
    eng, runner, clock = make_with_clock(pool_tokens=512, max_batch_tokens=64, prefill_chunk=16, prefix_share=True)
    stem = [t % 97 for t in range(7, 47)]  # 40 tokens: three portions of at most 16
    rids = [eng.add_request(stem + [i], greedy(3)) for i in (1, 2, 3)]
    other = eng.add_request([50, 51, 52], greedy(3))
    while eng.has_unfinished():
        eng.step()
        runner.cache.check()
    prefills = [c for call in runner.model.calls for c in call if c[2] > 1]
    assert prefills[:3] == [(rids[0], 0, 16), (rids[0], 16, 16), (rids[0], 32, 9)], "the first computes the whole prompt"
    assert [eng.requests[r].cached_tokens for r in rids] == [0, 40, 40], "the others waited and took its pages over"
    assert [c for c in prefills if c[0] in rids[1:]] == [], "and computed only their own last token"
    for rid, i in zip(rids, (1, 2, 3)):
        assert eng.requests[rid].output == expected_generation(stem + [i], 3, 97)[0]
    assert eng.requests[other].output == expected_generation([50, 51, 52], 3, 97)[0]


def test_random_workloads_with_everything_at_once():
    """Classes, aging, displacement, cancellation, sharing, eviction and preemption together, on random settings:
    no answer changes, the cache's books balance after every pass, nothing is held at the end but what the tree keeps."""
    for seed in range(40):
        rng = random.Random(1000 + seed)
        clock = Clock()
        share = rng.random() < 0.7
        runner = FakeRunner(page_size=rng.choice([2, 4, 8]), pool_tokens=rng.choice([48, 64, 96, 160]),
                            max_requests=rng.choice([2, 3, 4]), prefix_share=share, read_pages=True)
        cfg = SchedulerConfig(max_batch_tokens=rng.choice([8, 24, 64]), prefill_chunk=rng.choice([4, 16, 64]),
                              min_chunk=rng.choice([1, 4, 16]), max_running=rng.choice([0, 1, 2]), max_positions=256,
                              age_promote_s=rng.choice([0, 0.5, 5]), background_chunk_cap=rng.choice([0, 4]),
                              preempt=rng.random() < 0.8)
        eng = Engine(runner, cfg, sample_fn=argmax_sampler, clock=clock)
        stems = [[rng.randrange(97) for _ in range(rng.randrange(4, 30))] for _ in range(2)]
        todo = [(rng.choice(stems)[:rng.randrange(1, 30)] + [rng.randrange(97) for _ in range(rng.randrange(1, 8))],
                 greedy(rng.randrange(1, 25)), rng.choice([0, 0, 1])) for _ in range(rng.randrange(2, 10))]
        rids, passes = {}, 0
        while todo or eng.has_unfinished():
            if todo and rng.random() < 0.4:
                p, sp, pr = todo.pop(0)
                try:
                    rids[eng.add_request(p, sp, priority=pr)] = (p, sp)
                except ValueError:
                    pass  # a prompt the pool can never hold is refused at submit
            clock.now += rng.random() * 0.3
            if rids and rng.random() < 0.03:
                eng.cancel(rng.choice(list(rids)))
            eng.step()
            runner.cache.check()
            passes += 1
            assert passes < 5000, f"seed {seed}: no progress"
        for rid, (p, sp) in rids.items():
            r = eng.requests[rid]
            assert r.output == expected_generation(p, sp.max_tokens, 97)[0][:len(r.output)], f"seed {seed} request {rid}"
            assert r.finish_reason in ("length", "cancelled")
        st = runner.cache.stats()
        assert st["groups"][0]["used"] == (st["prefix"]["nodes"] if share else 0), f"seed {seed}"


# ------------------------------------------------------------------------------------------ lookahead

def select_on_device(logits, states):
    import torch
    return torch.argmax(logits, dim=-1).to(torch.int32)


def make_ahead(eos=(), **kw):
    runner = FakeRunner(page_size=kw.pop("page_size", 4), pool_tokens=kw.pop("pool_tokens", 256),
                        max_requests=kw.pop("max_requests", 4), prefix_share=kw.pop("prefix_share", False), read_pages=True)
    kw.setdefault("max_positions", 256)
    return Engine(runner, SchedulerConfig(**kw), eos_token_ids=eos, sample_fn=argmax_sampler, select_fn=select_on_device), runner


def test_lookahead_reads_tokens_one_pass_late_and_changes_nothing():
    eng, runner = make_ahead(max_batch_tokens=64, prefill_chunk=64)
    prompts = [[5, 6, 7, 8], [1, 2, 3], [9]]
    seen = []
    eng.on_token = lambda rid, tok: seen.append((rid, tok))
    res = eng.generate(prompts, [greedy(12), greedy(7), greedy(12)])
    for p, r, n in zip(prompts, res, (12, 7, 12)):
        assert r.tokens == expected_generation(p, n, 97)[0] and r.finish_reason == "length"
    assert eng.lookahead_passes >= 8, "most decode passes were launched before the tokens of the pass before were read"
    assert [t for rid, t in seen if rid == 0] == res[0].tokens
    # the tokens a pass was fed on the device are the ones the pass before sampled
    assert runner.model.calls[0] == [(0, 0, 4), (1, 0, 3), (2, 0, 1)] and runner.model.calls[3] == [(0, 6, 1), (1, 5, 1), (2, 3, 1)]
    runner.cache.check()
    assert runner.cache.stats()["groups"][0]["used"] == 0


def test_lookahead_with_stop_tokens_arrivals_and_cancellation():
    rng = random.Random(3)
    stops = 0
    for trial in range(30):
        eos = tuple(rng.sample(range(97), rng.choice([0, 3, 10])))
        eng, runner = make_ahead(eos=eos, pool_tokens=rng.choice([64, 128, 256]), page_size=rng.choice([2, 4, 8]),
                                 max_batch_tokens=rng.choice([8, 24, 64]), prefill_chunk=rng.choice([4, 16, 64]),
                                 min_chunk=rng.choice([1, 4]), max_requests=rng.choice([2, 4]), prefix_share=rng.random() < 0.5)
        todo = [([rng.randrange(97) for _ in range(rng.randrange(1, 30))], greedy(rng.randrange(1, 25))) for _ in range(rng.randrange(1, 8))]
        rids, cancelled = {}, set()
        while todo or eng.has_unfinished():
            if todo and rng.random() < 0.3:
                p, sp = todo.pop(0)
                rids[eng.add_request(p, sp)] = (p, sp)
            if rids and rng.random() < 0.02:
                rid = rng.choice(list(rids))
                eng.cancel(rid)
                cancelled.add(rid)
            eng.step()
            runner.cache.check()
        for rid, (p, sp) in rids.items():
            r = eng.requests[rid]
            exp, why = expected_generation(p, sp.max_tokens, 97, eos)
            if r.finish_reason == "cancelled":
                assert rid in cancelled and r.output == exp[:len(r.output)]
            elif r.stats["preemptions"] == 0 or r.finish_reason == "stop":
                assert (r.output, r.finish_reason) == (exp, why) or (r.finish_reason == "length" and r.output == exp[:len(r.output)])
            stops += r.finish_reason == "stop"
        st = runner.cache.stats()
        assert st["groups"][0]["used"] == (st["prefix"]["nodes"] if st["prefix"] else 0)
    assert stops > 10


# ------------------------------------------------------------------------------------------------ the step's own failures


def test_a_step_that_fails_in_the_model_leaves_the_cache_as_it_was():
    """An error raised by the model (a kernel that refuses, no memory during a capture) after the pages were begun:
    the pages go back, a request the step opened is closed, and the same step can be run again."""
    from jllm_serve_amd.engine.step import StepEntry
    runner = FakeRunner(page_size=4, pool_tokens=32, max_requests=3)
    runner.step([StepEntry("old", [1, 2, 3, 4, 5], [4])])
    used = [g.pool.used_pages for g in runner.cache.groups]
    real_forward = runner.model.forward

    def failing(step, slots):
        raise RuntimeError("the model failed")

    runner.model.forward = failing
    with pytest.raises(RuntimeError, match="the model failed"):
        runner.step([StepEntry("old", [6, 7, 8, 9], [3]), StepEntry("new", [1] * 9, [8])])
    runner.cache.check()
    assert [g.pool.used_pages for g in runner.cache.groups] == used
    assert runner.cache.length("old") == 5 and not runner.cache.has("new")
    assert len(runner.cache.table("old", 0)) == 2
    runner.model.forward = real_forward
    out = runner.step([StepEntry("old", [6, 7, 8, 9], [3]), StepEntry("new", [1] * 9, [8])])
    assert out.shape[0] == 2 and runner.cache.length("old") == 9 and runner.cache.length("new") == 9
    runner.cache.check()


def test_a_runner_cannot_hold_more_positions_than_the_model_was_built_for():
    """The position tables have one row per position of the model's build; the positions of a step live on the device."""
    class Build:
        max_positions = 64

    runner = FakeRunner(max_positions=64)
    runner.model.build = Build()
    from jllm_serve_amd.engine.step import ModelRunner
    ModelRunner(runner.model, runner.cache, 64)
    with pytest.raises(ValueError, match="built for 64"):
        ModelRunner(runner.model, runner.cache, 65)
    # and the scheduler's limit follows the runner's
    eng = Engine(runner, SchedulerConfig(max_positions=4096))
    assert eng.config.max_positions == 64


def test_captured_batch_sizes_end_with_the_full_batch():
    from jllm_serve_amd.engine.graphs import batch_buckets
    assert batch_buckets(1) == [1]
    assert batch_buckets(6) == [1, 2, 4, 6]
    assert batch_buckets(8) == [1, 2, 4, 8]
    assert batch_buckets(64) == [1, 2, 4, 8, 16, 32, 64]
    assert batch_buckets(3) == [1, 2, 3] and batch_buckets(0) == [1]


def test_a_session_at_its_limit_waits_although_places_are_free():
    """The reference's vector (T/SchedulerPolicyTest.java:233-246; engine/Admission.java:184-189, :225): three places,
    one request per session at a time. alice's second request waits while bob's is admitted beside her first, and goes
    when her first ends; a request without a session is never held back; a held-back request displaces nobody."""
    eng, runner, clock = make_with_clock(pool_tokens=512, max_requests=3, session_max_running=1, max_batch_tokens=64)
    eng.add_request([1, 2, 3], greedy(3), rid="a1", session="alice")
    eng.add_request([4, 5, 6], greedy(6), rid="a2", session="alice")
    eng.add_request([7, 8, 9], greedy(6), rid="b1", session="bob")
    eng.add_request([9, 9], greedy(6), rid="free")
    eng.step()
    running = {r.rid for r in eng.scheduler.running}
    assert running == {"a1", "b1", "free"}, running
    assert [r.rid for r in eng.scheduler.waiting] == ["a2"]
    while eng.requests["a1"].status != "finished":
        assert "a2" not in {r.rid for r in eng.scheduler.running}, "alice's second request ran beside her first"
        eng.step()
    eng.step()
    assert "a2" in {r.rid for r in eng.scheduler.running}, "and goes when her first request ends"
    while eng.has_unfinished():
        eng.step()
    for rid, prompt, n in (("a1", [1, 2, 3], 3), ("a2", [4, 5, 6], 6), ("b1", [7, 8, 9], 6), ("free", [9, 9], 6)):
        assert eng.requests[rid].output == expected_generation(prompt, n, 97)[0]
    runner.cache.check()
    # every place taken by background work of other sessions, alice's interactive request held back by her own
    # running one: nobody is displaced for it
    eng, runner, clock = make_with_clock(pool_tokens=512, max_requests=2, session_max_running=1, max_batch_tokens=64)
    eng.add_request([1, 2, 3], greedy(20), rid="a1", session="alice")
    eng.add_request([4, 5, 6], greedy(20), rid="bg", priority="background", session="carol")
    eng.step()
    eng.add_request([7, 8], greedy(2), rid="a2", session="alice")
    for _ in range(5):
        eng.step()
    assert eng.scheduler.displaced == 0 and {r.rid for r in eng.scheduler.running} == {"a1", "bg"}
    # without the limit the same arrival displaces the background request
    eng, runner, clock = make_with_clock(pool_tokens=512, max_requests=2, max_batch_tokens=64)
    eng.add_request([1, 2, 3], greedy(20), rid="a1", session="alice")
    eng.add_request([4, 5, 6], greedy(20), rid="bg", priority="background", session="carol")
    eng.step()
    eng.add_request([7, 8], greedy(2), rid="a2", session="alice")
    eng.step()
    assert eng.scheduler.displaced == 1


def test_a_displaced_request_still_holds_its_session_place():
    """engine/Admission.java:183-189 counts every slot of a session that is not idle, the paused ones included: a
    background request that was displaced and waits to go on still holds its session's one place. An interactive
    request of that session that arrives meanwhile neither takes a free place nor displaces anybody; it runs when the
    displaced request has gone on and ended."""
    eng, runner, clock = make_with_clock(pool_tokens=512, max_requests=2, max_running=2, session_max_running=1,
                                         max_batch_tokens=64)
    eng.add_request([1, 2, 3], greedy(12), rid="c1", priority="background", session="carol")
    eng.add_request([4, 5, 6], greedy(8), rid="d1", priority="background", session="dave")
    eng.step()
    eng.add_request([7, 8], greedy(3), rid="i1")  # interactive: displaces the background request that started last
    eng.step()
    assert eng.scheduler.displaced == 1 and [r.rid for r in eng.scheduler.waiting if r.preemptions > 0] == ["d1"]
    eng.add_request([9, 9, 9], greedy(2), rid="d2", session="dave")  # interactive, of the displaced request's session
    seen_d1 = False
    while eng.requests["d1"].status != "finished":
        eng.step()
        running = {r.rid for r in eng.scheduler.running}
        assert "d2" not in running, "dave's second request ran while his first held the session's place"
        seen_d1 = seen_d1 or "d1" in running
    assert seen_d1 and eng.scheduler.displaced == 1, "the held-back request displaced nobody"
    while eng.has_unfinished():
        eng.step()
    for rid, prompt, n in (("c1", [1, 2, 3], 12), ("d1", [4, 5, 6], 8), ("i1", [7, 8], 3), ("d2", [9, 9, 9], 2)):
        assert eng.requests[rid].output == expected_generation(prompt, n, 97)[0]
    runner.cache.check()
