"""Logits at the layer widths the benchmarks run: one or two layers of the Qwen3-8B, 14B and 32B shapes with the
real vocabulary (151,936) and random weights, replayed in the four ways of the trace tests (whole; all but the last
32 tokens in one step, then one by one; portions of changing size down to two tokens; mixed with other requests
on a pool of exactly the pages the busiest step needs, with the free pages reordered before every step), in
float32 and bfloat16, against the plain implementation in float32.

The weights come from the engine's random source on the GPU (no model folder of several gigabytes is written);
the plain side gets the same tensors by name. The replay goes through engine/trace.py's TraceRunner, which is
what bin/trace_run loops around. In bfloat16 every product and every attention call must have taken the
matrix-core kernel meant for it: nothing may have fallen back to the general kernels.
"""
import time
import zlib

import numpy as np
import pytest
import torch

import replay

pytestmark = pytest.mark.gpu

VOCAB = 151936
SHAPES = {  # layers here, hidden, heads, kv heads, head size, intermediate
    "8b": (2, 4096, 32, 8, 128, 12288),
    "14b": (1, 5120, 40, 8, 128, 17408),
    "32b": (1, 5120, 64, 8, 128, 25600),
}
PAGE = 16
LENGTHS = [7, 40, 150, 300]


def shape_config(name):
    L, d, H, Hkv, hd, F = SHAPES[name]
    return dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=L, hidden_size=d,
                num_attention_heads=H, num_key_value_heads=Hkv, head_dim=hd, intermediate_size=F, vocab_size=VOCAB,
                rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=name != "8b", max_position_embeddings=512)


def tokens(name, n, seed=0):
    g = torch.Generator().manual_seed(zlib.crc32(f"{name}/{n}/{seed}".encode()))
    return torch.randint(0, VOCAB, (n,), generator=g).tolist()


def build_trace(name):
    t = replay.Trace(page=PAGE)
    toks = {f"r{n}": tokens(name, n) for n in LENGTHS}
    longest = toks[f"r{LENGTHS[-1]}"]
    replay.whole(t, "whole", longest)
    replay.tail_one_by_one(t, "tail", longest)
    replay.portions(t, "cut", longest, sizes=(7, 2, 16, 3, 2, 65, 5, 2, 130, 9))
    more = dict(toks)
    more["x1"] = tokens(name, 45, seed=1)
    more["x2"] = tokens(name, 2, seed=2)
    replay.mixed(t, more, seed=len(name))
    return t, {"whole": longest, "tail": longest, "cut": longest, **more}


@pytest.fixture(scope="module", params=sorted(SHAPES))
def shape(request):
    """The shape's config, a weight source on the GPU, and plain float32 logits of every request of its trace."""
    from plain import qwen3_plain
    from jllm_serve_amd.weights.random_init import random_source
    name = request.param
    cfg = shape_config(name)
    t0 = time.time()
    source = random_source(cfg, seed=len(name), device="cuda")
    weights = {n: source.get(n).float().cpu() for n in source.names()}
    trace, req_tokens = build_trace(name)
    plain = {}
    for rid, tk in req_tokens.items():
        key = tuple(tk)
        if key not in plain:
            plain[key] = qwen3_plain.forward(cfg, weights, tk, dtype=torch.float32).numpy()
    del weights
    print(f"{name}: weights and {len(plain)} plain forwards in {time.time() - t0:.0f} s", flush=True)
    return name, cfg, source, trace, req_tokens, plain


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_real_widths(shape, dtype):
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import build_model
    from jllm_serve_amd.engine.trace import TraceRunner
    from jllm_serve_amd.kernels import ops
    name, cfg, source, trace, req_tokens, plain = shape
    print(f"real widths {name} {dtype}: {len(trace.steps)} steps, pool of {trace.peak} tokens", flush=True)
    model = build_model(parse_config(cfg), source, dtype, torch.device("cuda"), max(512, trace.peak))
    tr = TraceRunner(None, dtype, trace.peak, page_size=PAGE, max_live=4, shuffle_free=3, model=model)
    ops.reset_stats()
    rows = agree = 0
    worst = 0.0
    worst_of = {}
    kept = {}  # float32: (request, position) -> logits of the requests that run the same tokens in different cuts
    for rec in trace.steps:
        logits = tr.step(rec)
        if rec["step"] not in trace.rows:
            assert logits is None
            continue
        got = logits.cpu().numpy()
        for i, (rid, pos) in enumerate(trace.rows[rec["step"]]):
            ref = plain[tuple(req_tokens[rid])][pos]
            m = float(np.abs(ref).max())
            tol = 1e-4 * m + 1e-5 if dtype == "float32" else 1.5e-2 * m
            err = float(np.abs(got[i] - ref).max())
            worst = max(worst, err / tol)
            worst_of[rid] = max(worst_of.get(rid, 0.0), round(err / tol, 3))
            assert err <= tol, f"{name} {dtype}: step {rec['step']} request {rid} position {pos}: |diff| {err:.3g} > {tol:.3g}"
            if dtype == "float32" and rid in ("whole", "tail", "cut"):
                kept[(rid, pos)] = got[i].copy()
            best = int(got[i].argmax())
            same = best == int(ref.argmax())
            agree += same
            rows += 1
            if dtype == "float32":  # equal argmax, unless the plain side's two best are closer than the bound itself
                assert same or ref[best] >= ref.max() - tol, f"{name}: argmax differs at request {rid} position {pos}"
    tr.runner.cache.check()
    st = ops.stats()
    print(f"real widths {name} {dtype}: {rows} rows, worst error / tolerance {worst:.3f}, argmax agreement "
          f"{agree}/{rows} = {agree / rows:.4f}; per request {worst_of}; kernels {st['ran']}", flush=True)
    if dtype == "bfloat16":
        assert not st["general"], f"a product or attention call fell back to the general kernel: {st}"
        # near-ties among 151,936 random logits flip under bfloat16 rounding; far fewer rows agree when a kernel is wrong
        assert agree / rows >= 0.9
    else:
        assert not st["ran"], f"the float32 run used a reduced-precision kernel: {st}"
        # the 32-bit kernels add in an order that follows from a row's own position: cutting changes no bit
        for pos in range(len(req_tokens["whole"])):
            for other in ("tail", "cut"):
                assert np.array_equal(kept[("whole", pos)], kept[(other, pos)]), \
                    f"{name}: position {pos} of '{other}' differs in bits from the whole prompt's"


def test_bfloat16_error_is_what_its_rounding_points_give():
    """Is the bfloat16 path as exact as bfloat16 allows? The plain formulas in float64 with a rounding to bfloat16 at
    exactly the places where the engine stores bfloat16 (normed rows, projection outputs, q and k after norm and
    rotation, probabilities as they enter the weighted sum, attention output, the gated product) make an error
    against the unrounded formulas; the engine's error against the same must be of that size, not larger: a kernel
    that rounds twice, sums in bfloat16 or drops low bits would show here although it stays inside the 1.5 % bound.
    Two layers at the 8B widths, 300 positions, the real vocabulary."""
    import math
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import build_model, build_runner
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights.random_init import random_source
    dev = torch.device("cuda")
    cfg = shape_config("8b")
    src = random_source(cfg, seed=2, device="cuda")
    w = {n: src.get(n) for n in src.names()}
    T = 300
    toks = tokens("8b", T, seed=9)
    H, Hkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]

    def forward(r):  # r: what happens at a place where the engine stores bfloat16
        f = lambda n: w[n].to(torch.float64)
        x = f("model.embed_tokens.weight")[toks]
        inv = 1.0 / (cfg["rope_theta"] ** (torch.arange(0, hd // 2, device=dev, dtype=torch.float64) * 2 / hd))
        ang = torch.arange(T, device=dev, dtype=torch.float64)[:, None] * inv[None, :]
        cos, sin = torch.cos(ang).float().double()[:, None, :], torch.sin(ang).float().double()[:, None, :]

        def norm(v, g):
            return v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * g

        def rope(v):
            a, b = v[..., :hd // 2], v[..., hd // 2:]
            return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
        mask = torch.triu(torch.ones(T, T, dtype=torch.bool, device=dev), 1)
        for l in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{l}."
            xb = r(norm(x, f(p + "input_layernorm.weight")))
            q = r(xb @ f(p + "self_attn.q_proj.weight").T).view(T, H, hd)
            k = r(xb @ f(p + "self_attn.k_proj.weight").T).view(T, Hkv, hd)
            v = r(xb @ f(p + "self_attn.v_proj.weight").T).view(T, Hkv, hd)
            q = r(rope(norm(q, f(p + "self_attn.q_norm.weight"))))
            k = r(rope(norm(k, f(p + "self_attn.k_norm.weight"))))
            att = torch.zeros(T, H, hd, device=dev, dtype=torch.float64)
            for h in range(H):
                sc = ((q[:, h] @ k[:, h // (H // Hkv)].T) / math.sqrt(hd)).masked_fill(mask, float("-inf"))
                e = torch.exp(sc - sc.max(-1, keepdim=True).values)
                att[:, h] = (r(e) @ v[:, h // (H // Hkv)]) / e.sum(-1, keepdim=True)
            x = x + r(att.reshape(T, H * hd)) @ f(p + "self_attn.o_proj.weight").T
            xb = r(norm(x, f(p + "post_attention_layernorm.weight")))
            g, u = xb @ f(p + "mlp.gate_proj.weight").T, xb @ f(p + "mlp.up_proj.weight").T
            x = x + r(g / (1 + torch.exp(-g)) * u) @ f(p + "mlp.down_proj.weight").T
        return r(norm(x, f("model.norm.weight"))) @ f("lm_head.weight").T

    exact = forward(lambda t: t)
    rounded = forward(lambda t: t.to(torch.bfloat16).to(torch.float64))
    model = build_model(parse_config(cfg), src, "bfloat16", dev, 512)
    runner = build_runner(model, page_size=PAGE, pool_tokens=512, max_requests=1)
    got = runner.step([StepEntry("r", toks, list(range(T)))]).double()

    def rms(t):
        return float(t.pow(2).mean().sqrt())
    want_rms, got_rms = rms(rounded - exact), rms(got - exact)
    want_max, got_max = float((rounded - exact).abs().max()), float((got - exact).abs().max())
    print(f"bfloat16 rounding points: rms error {want_rms:.5f} (largest {want_max:.4f}); engine: {got_rms:.5f} ({got_max:.4f}); "
          f"engine against the rounded formulas: rms {rms(got - rounded):.5f}", flush=True)
    assert got_rms <= 1.15 * want_rms, f"the engine's bfloat16 error {got_rms} is larger than its rounding points explain ({want_rms})"
    assert got_max <= 1.5 * want_max


def test_preemption_and_recomputation_at_real_widths():
    """Generation through the engine at the 14B widths (40 query heads over 8, the real vocabulary) on a pool so small
    that requests are preempted and computed again, against the same requests on a pool that holds them all: the same
    tokens (float32: every sum has one fixed order), portions beside decoding rows, pages reused, the pool's books
    whole at the end."""
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_model, build_runner
    from jllm_serve_amd.sampling import SamplingParams
    from jllm_serve_amd.weights.random_init import random_source
    cfg = shape_config("14b")
    source = random_source(cfg, seed=4, device="cuda")
    model = build_model(parse_config(cfg), source, "float32", torch.device("cuda"), 512)
    prompts = [tokens("14b", n, seed=20 + n) for n in (150, 90, 40, 7)]
    params = SamplingParams(temperature=0.7, top_p=0.9, seed=11, max_tokens=24)

    def run(pool_tokens):
        runner = build_runner(model, page_size=PAGE, pool_tokens=pool_tokens, max_requests=4)
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=96, prefill_chunk=64, max_positions=512), eos_token_ids=())
        res = eng.generate(prompts, params)
        runner.cache.check()
        assert all(g.pool.used_pages == 0 for g in runner.cache.groups)
        return [r.tokens for r in res], eng.scheduler.preemptions

    roomy, none = run(1024)
    tight, some = run(272)  # the four requests would hold 150 + 90 + 40 + 7 + 4 * 24 = 383 positions at their ends
    print(f"preemptions: {none} with room, {some} on the tight pool", flush=True)
    assert none == 0 and some > 0, "the tight pool was meant to be too small"
    assert tight == roomy
    assert all(len(t) == 24 for t in roomy)
