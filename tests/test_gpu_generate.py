"""Generation through the entry points (Python API, command line) against the plain implementation, the selection
kernel against the plain sampler, temperature runs that must not depend on batching or preemption."""
import json
import os
import random
import subprocess
import sys

import pytest
import torch

import tiny
from plain import qwen3_plain as P
from plain import sampler_plain as S

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def make_engine(folder, dtype, page, **kw):
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    model = load_model(folder, dtype, torch.device(DEV), max_positions=kw.pop("ctx", 256))
    runner = build_runner(model, page_size=page, pool_tokens=kw.pop("pool", 1024), max_requests=kw.pop("slots", 4))
    sc = SchedulerConfig(max_batch_tokens=kw.pop("budget", 64), prefill_chunk=kw.pop("chunk", 32),
                         max_positions=runner.max_positions, **kw)
    return Engine(runner, sc, eos_token_ids=model.config.eos_token_ids)


def test_greedy_generation_matches_plain(model_folders):
    """Configuration A's workload: prompts of 5 / 17 / 33 tokens, 16 greedy tokens each, through Engine.generate."""
    from jllm_serve_amd.sampling import SamplingParams
    cfg, _, page = tiny.CONFIGS["A"]
    w = tiny.load_weights(model_folders["A"])
    prompts = [tiny.prompt("A", n) for n in (5, 17, 33)]
    want = [P.greedy(cfg, w, p, 16) for p in prompts]
    eng = make_engine(model_folders["A"], "float32", page, ctx=128)
    res = eng.generate(prompts, SamplingParams.greedy_params(max_tokens=16))
    assert [r.tokens for r in res] == want and all(r.finish_reason == "length" for r in res)
    assert all(r.stats["generated_tokens"] == 16 and r.stats["prompt_tokens"] == len(p) for r, p in zip(res, prompts))
    eng16 = make_engine(model_folders["A"], "bfloat16", page, ctx=128)
    res16 = eng16.generate(prompts, SamplingParams.greedy_params(max_tokens=16))
    agree = sum(a == b for r, wnt in zip(res16, want) for a, b in zip(r.tokens, wnt))
    assert all(r.tokens[0] == wnt[0] for r, wnt in zip(res16, want)) and agree >= 24, f"bfloat16 agrees on {agree}/48 tokens"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_lookahead_gives_the_same_tokens(dtype, model_folders):
    """Decode passes launched before the tokens of the pass before are read (their ids fed on the device, through
    captured steps in bfloat16): the same tokens as with every pass read at once, greedy and with temperature, top-k and top-p, with a
    stop token that ends one request early."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    cfg, _, page = tiny.CONFIGS["D"]
    prompts = [tiny.prompt("D", n, seed=7) for n in (5, 33, 70)]
    params = [SamplingParams.greedy_params(max_tokens=40), SamplingParams(temperature=0.8, top_k=20, top_p=0.95, seed=7, max_tokens=25),  # top-k and top-p inside the look-ahead too
              SamplingParams.greedy_params(max_tokens=40)]
    model = load_model(model_folders["D"], dtype, torch.device(DEV), max_positions=256)

    def run(lookahead, eos=()):
        runner = build_runner(model, page_size=page, pool_tokens=1024, max_requests=4)
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=128, prefill_chunk=64, max_positions=256), eos_token_ids=eos,
                     lookahead=lookahead)
        res = eng.generate(prompts, params)
        runner.cache.check()
        return [(r.tokens, r.finish_reason) for r in res], eng
    plain_way, e0 = run(False)
    ahead, e1 = run(True)
    assert e0.lookahead_passes == 0 and e1.lookahead_passes >= 30
    assert ahead == plain_way
    stop = plain_way[0][0][10]  # a token the first request generates: it now ends there
    a, _ = run(True, eos=(stop,))
    b, _ = run(False, eos=(stop,))
    assert a == b and a[0][1] == "stop" and len(a[0][0]) <= 10


def test_command_line_run(model_folders):
    cfg, _, page = tiny.CONFIGS["B"]
    w = tiny.load_weights(model_folders["B"])
    prompt = tiny.prompt("B", 9)
    want = P.greedy(cfg, w, prompt, 8)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "jllm"), "run", "--model", model_folders["B"], "--dtype", "float32",
           "--prompt", " ".join(map(str, prompt)), "--temp", "0", "--max-tokens", "8", "--page-size", str(page),
           "--ctx", "128", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["tokens"] == want and out["finish_reason"] == "length"
    assert "finish=length" in r.stderr and "prompt tok" in r.stderr
    bad = subprocess.run(cmd[:3] + ["--no-such-option", "1"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2 and "unknown option" in bad.stderr


def test_selection_kernel_against_plain_sampler():
    from jllm_serve_amd.kernels import ops
    rng = random.Random(1)
    g = torch.Generator().manual_seed(0)
    cases = []
    for V in (301, 4096):
        for (t, k, p, mp) in ((0.0, 0, 1.0, 0.0), (0.8, 0, 1.0, 0.0), (0.7, 20, 0.95, 0.0), (1.3, 0, 0.9, 0.0), (1.0, 5, 1.0, 0.0),
                              (0.6, 20, 0.95, 0.05), (1.0, 1, 0.5, 0.0), (2.0, 0, 0.3, 0.2), (1.0, 10000, 0.8, 0.0)):
            for rep in range(6):
                cases.append((V, t, k, p, mp, rng.random()))
    for (t, k, p, mp) in ((0.0, 0, 1.0, 0.0), (0.8, 0, 1.0, 0.0), (0.7, 20, 0.95, 0.0), (1.3, 0, 0.9, 0.0), (0.6, 50, 0.9, 0.02), (1.0, 0, 1.0, 0.05)):
        for u in (0.0, rng.random(), rng.random(), 0.999999):  # a long row: every scan takes several turns
            cases.append((40003, t, k, p, mp, u))
    for (t, k, p, mp) in ((0.0, 0, 1.0, 0.0), (0.7, 20, 0.95, 0.0), (1.0, 0, 0.9, 0.0)):  # the real vocabulary, a few rows
        cases.append((151936, t, k, p, mp, rng.random()))
    for V in (301, 4096, 40003, 151936):
        rows = [c for c in cases if c[0] == V]
        logits = torch.randn(len(rows), V, generator=g) * 4
        logits[0, 5] = logits[0, 9] = logits[0].max() + 1  # a tie for the maximum: the lower index wins when greedy
        out = ops.sample(logits.to(DEV), torch.tensor([c[1] for c in rows], dtype=torch.float32, device=DEV),
                         torch.tensor([c[2] for c in rows], dtype=torch.int32, device=DEV),
                         torch.tensor([c[3] for c in rows], dtype=torch.float32, device=DEV),
                         torch.tensor([c[4] for c in rows], dtype=torch.float32, device=DEV),
                         torch.tensor([c[5] for c in rows], dtype=torch.float64, device=DEV)).tolist()
        assert out[0] == 5
        for i, c in enumerate(rows):
            want = S.sample(logits[i].double().tolist(), c[1], c[2], c[3], c[4], c[5])
            assert out[i] == want, f"row {i}: V={V} T={c[1]} top_k={c[2]} top_p={c[3]} min_p={c[4]} u={c[5]}"
        am = ops.argmax(logits.to(DEV)).tolist()
        assert am == [S.argmax(r.tolist()) for r in logits]


def test_selection_kernel_when_many_logits_are_equal():
    """The kernel finds its thresholds in a bucket of nearby logits gathered into a list; a bucket with more entries
    than the list holds (thousands of equal or nearly equal logits) goes the long way. Rows made so that the k-th
    largest entry, or the entry at which top-p is reached, lies in such a bucket, against the plain sampler."""
    from jllm_serve_amd.kernels import ops
    V = 20011
    g = torch.Generator().manual_seed(4)
    base = torch.randn(V, generator=g)
    rows, params = [], []

    def add(z, t, k, p, mp, u):
        rows.append(z.clone())
        params.append((t, k, p, mp, u))

    flat = torch.full((V,), 0.25)
    for u in (0.0, 0.37, 0.999):
        add(flat, 1.0, 0, 0.5, 0.0, u)                       # everything equal: top-p keeps all of it
        add(flat, 0.7, 3000, 0.9, 0.0, u)                    # and so does top-k (the equals of the k-th all stay)
    plateau = base.clone()
    plateau[100:6100] = float(base.max()) + 0.5              # 6,000 equal largest entries
    for u in (0.1, 0.8):
        add(plateau, 1.0, 50, 1.0, 0.0, u)                   # the k-th largest lies among them
        add(plateau, 1.0, 0, 0.3, 0.0, u)                    # top-p is reached among them
        add(plateau, 0.5, 7000, 0.95, 0.0, u)                # the k-th largest lies behind them, top-p among them
    near = base.clone()
    near[5000:11000] = float(base.max()) - 0.001 * torch.rand(6000, generator=g)  # 6,000 different ones in one bucket
    for u in (0.2, 0.6, 0.95):
        add(near, 0.9, 2500, 0.8, 0.0, u)
        add(near, 1.0, 0, 0.6, 0.01, u)
    logits = torch.stack(rows)
    f = lambda i, dt: torch.tensor([q[i] for q in params], dtype=dt, device=DEV)
    out = ops.sample(logits.to(DEV), f(0, torch.float32), f(1, torch.int32), f(2, torch.float32), f(3, torch.float32),
                     f(4, torch.float64)).tolist()
    for i, q in enumerate(params):
        want = S.sample(logits[i].double().tolist(), *q)
        assert out[i] == want, f"row {i}: T={q[0]} top_k={q[1]} top_p={q[2]} min_p={q[3]} u={q[4]}"


def test_selection_kernel_the_short_way_and_the_long_way():
    """With top_k up to 128, or top-p alone, the kernel first collects the few largest entries into a list (what
    reaches the smallest of top_k, or of 64, group maxima) and takes thresholds and the draw from it if it is whole and
    top-p is reached inside it; else buckets over the whole row and more scans. Rows made for each way, with ties at
    the k-th place and at the list's edge, against the plain sampler."""
    from jllm_serve_amd.kernels import ops
    V = 60013
    g = torch.Generator().manual_seed(9)
    rows, params = [], []

    def add(z, t, k, p, mp, u):
        rows.append(z.clone())
        params.append((t, k, p, mp, u))

    flat = torch.randn(V, generator=g) * 1.3
    peaked = torch.randn(V, generator=g) * 2.0
    peaked[torch.randperm(V, generator=g)[:40]] += 14.0  # 40 entries far above the rest
    dense = torch.randn(V, generator=g) * 0.3
    tied = flat.clone()
    top = torch.topk(tied, 30).indices
    tied[top[15:25]] = float(tied[top[15]])              # ten equal entries around the 20th place: all of them stay
    plateau = peaked.clone()
    plateau[1000:3200] = float(peaked.max()) - 3.0       # 2,200 equal entries among the largest: more than the list holds
    for u in (0.0, 0.31, 0.77, 0.999999):
        add(flat, 0.6, 20, 0.95, 0.0, u)     # the short way
        add(peaked, 0.6, 20, 0.95, 0.0, u)
        add(peaked, 1.0, 35, 1.0, 0.0, u)
        add(peaked, 1.5, 0, 0.9, 0.0, u)     # top-p alone, reached among the 40: the short way
        add(flat, 1.0, 0, 0.9, 0.0, u)       # top-p alone, reached thousands of entries down: the long way after all
        add(dense, 0.6, 20, 0.95, 0.0, u)
        add(tied, 0.6, 20, 0.95, 0.0, u)
        add(tied, 1.0, 20, 1.0, 0.1, u)
        add(plateau, 0.8, 60, 0.95, 0.0, u)  # the list overflows: the long way
        add(flat, 1.0, 128, 0.999, 0.0, u)   # the largest top_k that tries the list
        add(flat, 1.0, 129, 0.999, 0.0, u)   # the first that does not
        add(flat, 1.0, 3000, 1.0, 0.0, u)
        add(peaked, 0.7, 5, 0.5, 0.3, u)     # min-p cuts further
    logits = torch.stack(rows)
    f = lambda i, dt: torch.tensor([q[i] for q in params], dtype=dt, device=DEV)
    out = ops.sample(logits.to(DEV), f(0, torch.float32), f(1, torch.int32), f(2, torch.float32), f(3, torch.float32),
                     f(4, torch.float64)).tolist()
    for i, q in enumerate(params):
        want = S.sample(logits[i].double().tolist(), *q)
        assert out[i] == want, f"row {i}: T={q[0]} top_k={q[1]} top_p={q[2]} min_p={q[3]} u={q[4]}"
    small = torch.randn(3, 50, generator=g) * 2          # fewer entries than threads: some groups see nothing
    out = ops.sample(small.to(DEV), torch.full((3,), 0.8, device=DEV), torch.tensor([20, 45, 0], dtype=torch.int32, device=DEV),
                     torch.tensor([0.9, 1.0, 0.7], device=DEV), torch.zeros(3, device=DEV),
                     torch.tensor([0.2, 0.9, 0.5], dtype=torch.float64, device=DEV)).tolist()
    for i, (k, p, u) in enumerate(((20, 0.9, 0.2), (45, 1.0, 0.9), (0, 0.7, 0.5))):
        assert out[i] == S.sample(small[i].double().tolist(), 0.8, k, float(torch.tensor(p, dtype=torch.float32)), 0.0, u)


def test_argmax_of_long_rows_keeps_the_lower_index():
    """Rows as long as a real vocabulary go through two launches (runs of the row, then a pick among the candidates):
    the largest entry wins, the lowest index among equals, also when the equals lie in different runs, in one run,
    at the row's ends or everywhere."""
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    for V in (16384, 151936, 40001):
        logits = torch.randn(9, V, generator=g)
        top = float(logits.max()) + 1.0
        logits[0, V - 1] = top                               # the last entry
        logits[1, 0] = logits[1, V - 1] = top                # both ends
        logits[2, V // 2 + 7] = logits[2, V // 3] = top      # two runs, the later one written first
        logits[3, 100] = logits[3, 101] = logits[3, 99] = top  # neighbours in one run
        logits[4, :] = 0.25                                  # all equal: index 0
        logits[5, V // 32 * 5:] = top                        # equal from a run's start to the end
        logits[6, 1:] = -float("inf")                        # everything but one entry is -inf
        logits[7, :] = -float("inf")                         # nothing is finite: index 0
        wide = torch.zeros(9, V + 5)
        wide[:, :V] = logits
        got = ops.argmax(wide.to(DEV)[:, :V]).tolist()       # rows with a stride of their own
        want = [V - 1, 0, V // 3, 99, 0, V // 32 * 5, 0, 0, int(torch.argmax(logits[8]))]
        assert got == want, (V, got, want)


def test_logprob_kernel_against_plain():
    """Log-probabilities and alternatives of rows of other widths than the models', with ties for the largest
    logits (the lower index comes first) and a huge offset (the log-sum-exp must not overflow)."""
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    for V, top in ((301, 5), (4099, 20), (17, 17), (50, 0)):
        logits = torch.randn(6, V, generator=g) * 3
        logits[1] += 3000.0
        logits[2, 4] = logits[2, 11] = logits[2, 2] = logits[2].max() + 0.5
        tokens = torch.randint(0, V, (6,), generator=g, dtype=torch.int32)
        lp, ids, tlp = ops.token_logprobs(logits.to(DEV), tokens.to(DEV), top)
        for r in range(6):
            w_lp, w_ids, w_tlp = S.token_logprob(logits[r].double().tolist(), int(tokens[r]), top)
            assert abs(float(lp[r]) - w_lp) <= 1e-5 * max(1.0, abs(w_lp))
            assert ids[r].tolist() == w_ids
            assert torch.allclose(tlp[r].cpu().double(), torch.tensor(w_tlp, dtype=torch.float64), rtol=1e-5, atol=1e-5)
    with pytest.raises(ops.KernelError):
        ops.token_logprobs(torch.randn(2, 8, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV), 9)


def test_logprobs_through_the_engine(model_folders):
    """A request that asks for logprobs gets one entry per generated token, equal to the plain model's log-softmax at
    that position (32-bit run), also when the sampler changes the logits (penalties) and beside a request that did
    not ask."""
    from jllm_serve_amd.sampling import SamplingParams
    import math
    cfg, _, page = tiny.CONFIGS["B"]
    w = tiny.load_weights(model_folders["B"])
    prompts = [tiny.prompt("B", 9), tiny.prompt("B", 20)]
    eng = make_engine(model_folders["B"], "float32", page, ctx=128)
    asked = SamplingParams(temperature=0.0, top_k=0, top_p=1.0, max_tokens=6, repetition_penalty=1.3, logprobs=True, top_logprobs=3)
    res = eng.generate(prompts, [asked, SamplingParams.greedy_params(max_tokens=6)])
    assert res[1].logprobs is None and len(res[0].logprobs) == 6
    with pytest.raises(ValueError):
        res[1].cumulative_logprob()
    seq = list(prompts[0])
    total = 0.0
    for tok, lp in zip(res[0].tokens, res[0].logprobs):
        z = P.forward(cfg, w, seq)[-1].double().tolist()
        w_lp, w_ids, w_tlp = S.token_logprob(z, tok, 3)
        assert lp.token == tok and abs(lp.logprob - w_lp) <= 2e-4 and list(lp.top_tokens) == w_ids
        assert all(abs(a - b) <= 2e-4 for a, b in zip(lp.top_logprobs, w_tlp))
        total += lp.logprob
        seq.append(tok)
    assert math.isclose(res[0].cumulative_logprob(), total, rel_tol=1e-9)


def test_prompt_logprobs_through_the_engine(model_folders):
    """One entry per prompt token, the first None, each the plain model's log-softmax at the position before; the
    prompt is cut into portions, another request runs beside it, the pool is so small that the request is preempted
    and computed again (nothing is reported twice), and with prefix sharing on the whole prompt is still computed."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    cfg, _, page = tiny.CONFIGS["B"]
    w = tiny.load_weights(model_folders["B"])
    prompt = tiny.prompt("B", 37)
    z = P.forward(cfg, w, prompt).double()
    model = load_model(model_folders["B"], "float32", torch.device(DEV), max_positions=128)
    runner = build_runner(model, page_size=page, pool_tokens=6 * page, max_requests=3, prefix_share=True)
    eng = Engine(runner, SchedulerConfig(max_batch_tokens=24, prefill_chunk=10, min_chunk=2, max_positions=128))
    eng.generate([prompt], SamplingParams.greedy_params(max_tokens=1))  # leaves the prompt's pages in the tree
    asked = SamplingParams(temperature=0.0, top_k=0, top_p=1.0, max_tokens=30, prompt_logprobs=True, top_logprobs=2)
    other = SamplingParams.greedy_params(max_tokens=30)
    res = eng.generate([tiny.prompt("B", 21, seed=4), prompt], [other, asked])
    assert eng.scheduler.preemptions > 0 and res[1].stats["preemptions"] > 0, "the pool was meant to be too small"
    assert res[1].stats["cached_tokens"] == 0 or res[1].stats["preemptions"] > 0
    got = res[1].prompt_logprobs
    assert res[0].prompt_logprobs is None and len(got) == len(prompt) and got[0] is None
    for i in range(1, len(prompt)):
        w_lp, w_ids, w_tlp = S.token_logprob(z[i - 1].tolist(), prompt[i], 2)
        assert got[i].token == prompt[i] and abs(got[i].logprob - w_lp) <= 2e-4 and list(got[i].top_tokens) == w_ids
    assert res[1].tokens == P.greedy(cfg, w, prompt, 30)
    both = eng.generate_choices(prompt, SamplingParams(temperature=0.0, top_k=0, top_p=1.0, max_tokens=2, prompt_logprobs=True), n=2)
    assert both[1].prompt_logprobs is both[0].prompt_logprobs and len(both[0].prompt_logprobs) == len(prompt)
    assert both[0].stats["cached_tokens"] == 0 and both[1].stats["cached_tokens"] >= 2 * page


def test_penalty_kernel():
    from jllm_serve_amd.kernels import ops
    z = torch.tensor([2.0, -2.0, 1.0, 0.5, 0.25])
    row = z.clone().to(DEV)
    ops.adjust_logits(row, torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV), torch.tensor([0, 2, 1], dtype=torch.int32, device=DEV),
                      2.0, 0.5, 0.25, torch.tensor([3], dtype=torch.int32, device=DEV), torch.tensor([-100.0], device=DEV))
    want = S.apply_penalties(z.tolist(), seen={0, 1, 2}, generated={1: 2, 2: 1}, rep=2.0, pres=0.5, freq=0.25, bias={3: -100.0})
    assert torch.allclose(row.cpu(), torch.tensor(want))


def test_temperature_workload_is_reproducible_and_independent_of_batching(model_folders):
    """Configuration B's workload: prompts of 1 / 9 / 40 / 100 tokens, portions of 32 mixed with decode steps, 24
    tokens at temperature 0.8 with seed 7. Each request alone gives the same tokens as all four together, as a
    run with so few pages that requests are preempted and recomputed, and as the plain model + plain sampler
    driven with the same uniform numbers."""
    from jllm_serve_amd.sampling import SamplingParams, uniform
    cfg, _, page = tiny.CONFIGS["B"]
    folder = model_folders["B"]
    prompts = [tiny.prompt("B", n) for n in (1, 9, 40, 100)]
    params = SamplingParams(temperature=0.8, top_k=0, top_p=1.0, seed=7, max_tokens=24)
    together = make_engine(folder, "float32", page, budget=40, chunk=32).generate(prompts, params)
    alone = [make_engine(folder, "float32", page, budget=40, chunk=32).generate([p], params)[0] for p in prompts]
    assert [r.tokens for r in together] == [r.tokens for r in alone]
    tight = make_engine(folder, "float32", page, budget=40, chunk=32, pool=176, min_chunk=1)
    squeezed = tight.generate(prompts, params)
    assert tight.scheduler.preemptions > 0, "the pool of 176 positions cannot hold 1+9+40+100 prompts plus 24 tokens each"
    assert [r.tokens for r in squeezed] == [r.tokens for r in together]
    tight.runner.cache.check()
    # the plain model and sampler with the same uniform numbers
    w = tiny.load_weights(folder)
    for p, r in zip(prompts[:3], together[:3]):
        toks = list(p)
        for i in range(24):
            z = P.forward(cfg, w, toks)[-1].tolist()
            t = S.sample(z, 0.8, 0, 1.0, 0.0, uniform(7, i))
            assert t == r.tokens[i], f"prompt of {len(p)}: token {i}"
            toks.append(t)
    top = make_engine(folder, "float32", page).generate(prompts[:2], SamplingParams(temperature=0.8, seed=7, max_tokens=12))
    again = make_engine(folder, "float32", page).generate(prompts[:2], SamplingParams(temperature=0.8, seed=7, max_tokens=12))
    other = make_engine(folder, "float32", page).generate(prompts[:2], SamplingParams(temperature=0.8, seed=8, max_tokens=12))
    assert [r.tokens for r in top] == [r.tokens for r in again] != [r.tokens for r in other]


def test_eos_and_penalties_through_the_engine(model_folders):
    from jllm_serve_amd.sampling import SamplingParams
    cfg, _, page = tiny.CONFIGS["C"]  # eos_token_id = [7, 300]
    folder = model_folders["C"]
    w = tiny.load_weights(folder)
    prompt = tiny.prompt("C", 11)
    free = P.greedy(cfg, w, prompt, 12)
    eng = make_engine(folder, "float32", page, ctx=192)
    assert eng.eos == {7, 300}
    eng.eos = {free[5]}
    r = eng.generate([prompt], SamplingParams.greedy_params(max_tokens=12))[0]
    assert r.finish_reason == "stop" and r.tokens == free[:free.index(free[5])]
    r = eng.generate([prompt], SamplingParams.greedy_params(max_tokens=12, ignore_eos=True))[0]
    assert r.tokens == free
    # a repetition penalty through the engine equals the plain sampler applied to the plain logits
    eng.eos = set()
    pen = SamplingParams(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.8, presence_penalty=0.4, max_tokens=8)
    got = eng.generate([prompt], pen)[0].tokens
    toks, gen = list(prompt), {}
    for i in range(8):
        z = S.apply_penalties(P.forward(cfg, w, toks)[-1].tolist(), set(toks), gen, 1.8, 0.4, 0.0)
        t = S.argmax(z)
        assert got[i] == t
        toks.append(t)
        gen[t] = gen.get(t, 0) + 1
