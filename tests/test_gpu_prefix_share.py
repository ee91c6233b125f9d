"""Prefix sharing on the real cache: pages taken over from another request, a fork inside a page (rows copied by
the kernel), a rewind into a shared page, eviction; every logit against the plain implementation, which knows no
cache. The scenario is the reference's own (T/PagedKvChecks.java:184-226), with the plain model in the place of
its flat cache."""
import pytest
import torch

import tiny
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


def runner_for(folder, dtype, page, pool, slots=4):
    from jllm_serve_amd.engine import build_runner, load_model
    model = load_model(folder, dtype, torch.device(DEV), max_positions=128)
    return build_runner(model, page_size=page, pool_tokens=pool, max_requests=slots, graphs=False, prefix_share=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_adopt_fork_and_rewind(name, dtype, model_folders, plain_logits):
    from jllm_serve_amd.engine.step import StepEntry
    cfg, _, page = tiny.CONFIGS[name]
    V = cfg["vocab_size"]
    runner = runner_for(model_folders[name], dtype, page, pool=16 * page)
    cache = runner.cache
    tokens = tiny.prompt(name, 3 * page - 2)  # 46 with pages of 16: two full pages and most of a third
    fork_at = page + 5
    back_to = page + page // 2 + 1  # 25 with pages of 16
    other = tokens[:fork_at] + [(t + 101) % V for t in tokens[fork_at:]]

    def close_enough(got, ref, what):
        err = (got.cpu().double() - ref).abs().max()
        assert err <= tiny.tolerance(dtype, ref), f"{what}: {float(err)}"

    # a computes the prompt in two portions and publishes it
    cut = page + 4
    runner.step([StepEntry("a", tokens[:cut], [])])
    out = runner.step([StepEntry("a", tokens[cut:], range(len(tokens) - cut))])
    close_enough(out, plain_logits(name, tokens)[cut:], "the publisher itself")
    cache.publish("a", tokens)
    assert cache.published_pages("a") == 2
    # b takes the two full pages over and runs the rest
    cache.open("b")
    found = cache.match(tokens, len(tokens) - 1)
    assert (found.tokens, found.nodes, found.partial) == (2 * page, 2, 0)
    assert cache.adopt("b", tokens, 2 * page) == 2 * page
    assert cache.table("b", 0) == cache.table("a", 0)[:2]
    out = runner.step([StepEntry("b", tokens[2 * page:], range(len(tokens) - 2 * page))])
    close_enough(out, plain_logits(name, tokens)[2 * page:], "rows over adopted pages")
    # c shares one page and five rows of the next, which are copied into a page of its own
    cache.open("c")
    fm = cache.match(other, len(other) - 1)
    assert (fm.tokens, fm.nodes, fm.partial) == (fork_at, 1, 5)
    assert cache.adopt("c", other, fm.tokens) == fork_at
    assert cache.table("c", 0)[0] == cache.table("a", 0)[0] and cache.table("c", 0)[1] != cache.table("a", 0)[1]
    n_c = 8
    out = runner.step([StepEntry("c", other[fork_at:fork_at + n_c], range(n_c))])
    close_enough(out, plain_logits(name, other[:fork_at + n_c])[fork_at:], "a fork inside a page")
    # a rewinds into its second page, which b shares, and goes on with other tokens
    third = tokens[:back_to] + [(t + 7) % V for t in tokens[back_to:back_to + 6]]
    cache.truncate("a", back_to)
    out = runner.step([StepEntry("a", third[back_to:], range(6))])
    close_enough(out, plain_logits(name, third)[back_to:], "a rewind into a shared page")
    assert cache.table("a", 0)[1] != cache.table("b", 0)[1] and cache.stats()["prefix"]["copies_on_write"] == 2
    # b and c read their rows undisturbed
    nb, nc = (tokens[3] + 1) % V, (other[5] + 2) % V
    out = runner.step([StepEntry("b", [nb], [0]), StepEntry("c", [nc], [0])])
    close_enough(out[0:1], plain_logits(name, tokens + [nb])[-1:], "the sharer after the rewind")
    close_enough(out[1:2], plain_logits(name, other[:fork_at + n_c] + [nc])[-1:], "the fork after the rewind")
    cache.check()
    for rid in ("a", "b", "c"):
        cache.close(rid)
    cache.check()
    assert cache.stats()["groups"][0]["used"] == cache.stats()["prefix"]["nodes"] == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_shared_prompts_matches_plain(dtype, model_folders):
    """Requests that share a system prompt, through the engine, with a pool so small that cached pages are evicted
    and requests are preempted: greedy tokens as the plain implementation gives them (32-bit), and the same tokens
    with and without sharing (bfloat16: the first token, and at least half of the rest, as for bfloat16
    against the plain implementation elsewhere)."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    name = "B"
    cfg, _, page = tiny.CONFIGS[name]
    w = tiny.load_weights(model_folders[name])
    stem = tiny.prompt(name, 41)
    prompts = [stem + tiny.prompt(name, n, seed=n) for n in (3, 9, 1, 17)] + [stem[:30] + [5, 6]] + [stem + tiny.prompt(name, 3, seed=3)]
    want = [P.greedy(cfg, w, p, 12) for p in prompts]

    def run(share):
        model = load_model(model_folders[name], dtype, torch.device(DEV), max_positions=128)
        runner = build_runner(model, page_size=page, pool_tokens=11 * page, max_requests=3, prefix_share=share)
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=48, prefill_chunk=32, min_chunk=4, max_positions=128))
        first = eng.generate(prompts[:1], SamplingParams.greedy_params(max_tokens=12))
        rest = eng.generate(prompts[1:], SamplingParams.greedy_params(max_tokens=12))
        runner.cache.check()
        return first + rest, eng

    shared, eng = run(True)
    st = eng.runner.cache.stats()["prefix"]
    assert st["hits"] >= 4 and st["hit_tokens"] >= 4 * 32 and st["copies_on_write"] >= 1
    assert shared[5].stats["cached_tokens"] >= 32, "the first prompt again"
    if dtype == "float32":
        assert [r.tokens for r in shared] == want
    else:
        alone, _ = run(False)
        agree = sum(a == b for r, q in zip(shared, alone) for a, b in zip(r.tokens, q.tokens))
        assert all(r.tokens[0] == q.tokens[0] for r, q in zip(shared, alone)) and agree >= 6 * len(prompts), agree
