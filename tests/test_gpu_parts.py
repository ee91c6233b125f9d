"""Each part of a layer alone against the plain implementation: norm, position table, attention mixer, gated
feed-forward, the arranged block, the whole model; float32 and bfloat16; configurations B, C and D."""
import math

import pytest
import torch

import tiny
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def built(model_folders):
    """(name, dtype) -> (model, runner) on the GPU, built once."""
    from jllm_serve_amd.engine import build_runner, load_model
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            model = load_model(model_folders[name], dtype, torch.device(DEV), max_positions=512)
            cache[(name, dtype)] = (model, build_runner(model, page_size=tiny.CONFIGS[name][2], pool_tokens=1024,
                                                        max_requests=4, graphs=False))
        return cache[(name, dtype)]
    return get


def tol(dtype, ref):
    return (2e-5 if dtype == "float32" else 2.5e-2) * float(ref.abs().max()) + 1e-6


def step_context(runner, rid, n):
    from jllm_serve_amd.engine.step import StepEntry
    return runner.prepare([StepEntry(rid, [0] * n, list(range(n)))])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_norm_ffn_attention_block(name, dtype, built, model_folders):
    cfg_d = tiny.CONFIGS[name][0]
    cfg = P.read_config(cfg_d)
    w = tiny.load_weights(model_folders[name])
    model, runner = built(name, dtype)
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    torch.manual_seed(5)
    T = 37
    x = torch.randn(T, cfg["dim"]) * 0.7
    layer = model.layers[1]
    prefix = "model.layers.1"
    # norm
    got = layer.norm_in.forward(x.to(DEV)).float().cpu()
    ref = P.rmsnorm(x.double(), w[prefix + ".input_layernorm.weight"], cfg["eps"])
    assert (got.double() - ref).abs().max() <= tol(dtype, ref)
    # feed-forward: adds into the residual
    xb = (torch.randn(T, cfg["dim"]) * 0.5).to(act)
    res = torch.randn(T, cfg["dim"])
    want = res.double() + P.swiglu(xb.double(), w[prefix + ".mlp.gate_proj.weight"], w[prefix + ".mlp.up_proj.weight"],
                                   w[prefix + ".mlp.down_proj.weight"])
    r = res.clone().to(DEV)
    layer.ffn.forward(xb.to(DEV), r, None)
    assert (r.cpu().double() - want).abs().max() <= tol(dtype, want)
    # attention: a whole sequence from position 0 through the paged cache, then 5 more rows from the cache
    xb = (torch.randn(T + 5, cfg["dim"]) * 0.5).to(act)
    positions = torch.arange(T + 5)
    want = P.attention_block(xb.double(), w, prefix, cfg, 1, positions)
    slot = runner.cache.slots[1]
    out = []
    for n in (T, 5):
        ctx = step_context(runner, "att", n)
        res = torch.zeros(n, cfg["dim"], device=DEV)
        p0 = int(ctx.positions[0])
        layer.mixer.forward(xb[p0:p0 + n].to(DEV), res, ctx, slot)
        runner.cache.commit("att", n)
        out.append(res.cpu())
    runner.finish("att")
    got = torch.cat(out)
    assert (got.double() - want).abs().max() <= tol(dtype, want), "attention part through the cache"
    # the arranged block
    x0 = torch.randn(T, cfg["dim"]) * 0.7
    want = P.decoder_layer(x0.double(), w, 1, cfg, torch.arange(T))
    ctx = step_context(runner, "blk", T)
    xg = x0.clone().to(DEV)
    layer.forward(xg, ctx, slot)
    runner.finish("blk")
    assert (xg.cpu().double() - want).abs().max() <= tol(dtype, want)


@pytest.mark.parametrize("name", ["A", "C"])
def test_rotary_table_on_device(name, built):
    model, _ = built(name, "float32")
    cfg = P.read_config(tiny.CONFIGS[name][0])
    cos, sin, rdim = model.positions[0].rotary()
    pc, ps = P.rope_angles(torch.arange(cos.shape[0]), cfg["rotary_dim"], cfg["theta"], cfg["rope_scaling"], cfg["max_pos"])
    assert rdim == cfg["rotary_dim"] and torch.equal(cos.cpu(), pc) and torch.equal(sin.cpu(), ps)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_single_token_prompt(dtype, built, plain_logits):
    """The first positions of a sequence (position 0 is the rotation's identity and sees one key), one by one."""
    from jllm_serve_amd.engine.step import StepEntry
    for name in ("A", "B"):
        _, runner = built(name, dtype)
        toks = tiny.prompt(name, 6, seed=9)
        ref = plain_logits(name, toks)
        for i, t in enumerate(toks):
            got = runner.step([StepEntry("f", [t], [0])])[0].cpu().double()
            assert (got - ref[i]).abs().max() <= tiny.tolerance(dtype, ref[i]), f"{name} position {i}"
        runner.finish("f")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype, built, plain_logits):
    """A short prompt, then 300 tokens one by one (several splits of keys, many pages), teacher forced."""
    from jllm_serve_amd.engine import build_runner
    from jllm_serve_amd.engine.step import StepEntry
    model, _ = built("D", dtype)
    runner = build_runner(model, page_size=16, pool_tokens=384, max_requests=2)  # with captured decode steps in bfloat16
    toks = tiny.prompt("D", 330, seed=4)
    ref = plain_logits("D", toks)
    runner.step([StepEntry("long", toks[:30], [])])
    worst = 0.0
    for i in range(30, 330):
        got = runner.step([StepEntry("long", [toks[i]], [0])])[0].cpu().double()
        err = float((got - ref[i]).abs().max())
        worst = max(worst, err / tiny.tolerance(dtype, ref[i]))
        assert err <= tiny.tolerance(dtype, ref[i]), f"position {i}"
    runner.finish("long")
    if dtype == "bfloat16":
        assert runner.graphs is not None and runner.graphs.replays >= 300, "decode steps replay captured graphs"
    print(f"long decoding {dtype}: worst error / tolerance {worst:.3f}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_bias_is_inside_the_head_norm(dtype):
    """The engine's own kernels held to q = norm(W x + b): with eps -> 0, the q and k weights AND biases of every layer
    times 64 leave the logits where they were; the biases alone times 64 move them. (A bias added after the norm
    would turn this round.) Configuration C has biases, a window and partial sharing of heads."""
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import build_model, build_runner
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights import TensorSource
    from jllm_serve_amd.weights.random_init import random_source
    cfg_d = dict(tiny.TINY_C, rms_norm_eps=1e-12)
    src = random_source(cfg_d, seed=11)
    w = {n: src.get(n) for n in src.names()}
    both, bias_only = dict(w), dict(w)
    for n in ("q", "k"):
        for l in range(cfg_d["num_hidden_layers"]):
            key = f"model.layers.{l}.self_attn.{n}_proj."
            both[key + "weight"], both[key + "bias"] = w[key + "weight"] * 64, w[key + "bias"] * 64  # exact in bfloat16
            bias_only[key + "bias"] = w[key + "bias"] * 64
    toks = tiny.prompt("C", 40, seed=2)
    logits = []
    for weights in (w, both, bias_only):
        model = build_model(parse_config(cfg_d), TensorSource(weights), dtype, torch.device(DEV), 192)
        runner = build_runner(model, page_size=32, pool_tokens=192, max_requests=2, graphs=False)
        out = [runner.step([StepEntry("r", toks[:33], list(range(33)))])]
        out += [runner.step([StepEntry("r", [t], [0])]) for t in toks[33:]]  # the decode kernels as well
        logits.append(torch.cat(out).cpu().double())
    ref = P.forward(cfg_d, {k: v.double() for k, v in w.items()}, toks)
    assert (logits[0] - ref).abs().max() <= tiny.tolerance(dtype, ref)
    span = float(ref.abs().max())
    assert (logits[1] - logits[0]).abs().max() <= (1e-4 if dtype == "float32" else 1.5e-2) * span
    assert (logits[2] - logits[0]).abs().max() > 5e-2 * span


def test_captured_steps_are_dropped_and_recorded_again(built, plain_logits):
    """With room for one captured step only, steps of one, three and one requests in turn drop the recorded step of
    the other size every time and record it anew (its memory pool and pinned buffer go and come back); every row
    still matches the plain implementation, teacher forced."""
    from jllm_serve_amd.engine import build_runner
    from jllm_serve_amd.engine.graphs import DecodeGraphs
    from jllm_serve_amd.engine.step import StepEntry
    model, _ = built("D", "bfloat16")
    runner = build_runner(model, page_size=16, pool_tokens=512, max_requests=4, graphs=False)
    runner.graphs = DecodeGraphs(runner, 4, max_graphs=1)
    toks = {rid: tiny.prompt("D", n, seed=40 + n) for rid, n in (("ea", 60), ("eb", 45), ("ec", 52))}
    ref = {rid: plain_logits("D", t) for rid, t in toks.items()}
    at = {rid: len(t) - 14 for rid, t in toks.items()}
    runner.step([StepEntry(rid, toks[rid][:at[rid]], []) for rid in toks])
    for turn in range(12):
        rids = ["ea"] if turn % 2 == 0 else ["ea", "eb", "ec"]
        out = runner.step([StepEntry(rid, [toks[rid][at[rid]]], [0]) for rid in rids]).cpu().double()
        for i, rid in enumerate(rids):
            want = ref[rid][at[rid]]
            assert (out[i] - want).abs().max() <= tiny.tolerance("bfloat16", want), f"turn {turn}, request {rid}"
            at[rid] += 1
    assert runner.graphs.replays == 12 and runner.graphs.evictions >= 11 and len(runner.graphs.graphs) == 1
    for rid in toks:
        runner.finish(rid)
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context(dtype, model_folders, plain_logits):
    """A context far beyond the other tests' (2,300 positions, past the configuration's max_position_embeddings):
    the prompt in portions of up to 700 rows, another request's decode rows riding along, then single tokens
    across the 2,048 edge (where the captured decode steps change their bucket), teacher forced."""
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    model = load_model(model_folders["D"], dtype, torch.device(DEV), max_positions=2560)
    runner = build_runner(model, page_size=16, pool_tokens=2560 + 64, max_requests=2)
    toks = tiny.prompt("D", 2300, seed=6)
    ref = plain_logits("D", toks)
    side = tiny.prompt("D", 12, seed=7)
    side_ref = plain_logits("D", side)
    runner.step([StepEntry("side", side[:4], [])])
    pos, k = 0, 4
    for n in (700, 130, 3, 640, 512, 45):  # 2,030 rows in portions; the side request decodes beside them
        want = [0, n - 1]
        out = runner.step([StepEntry("long", toks[pos:pos + n], want), StepEntry("side", [side[k]], [0])]).cpu().double()
        for j, r in enumerate(want):
            assert (out[j] - ref[pos + r]).abs().max() <= tiny.tolerance(dtype, ref[pos + r]), f"portion at {pos}, row {r}"
        assert (out[2] - side_ref[k]).abs().max() <= tiny.tolerance(dtype, side_ref[k])
        pos += n
        k += 1
    runner.finish("side")
    assert pos == 2030

    def one_by_one(first, last):
        for i in range(first, last):
            got = runner.step([StepEntry("long", [toks[i]], [0])])[0].cpu().double()
            assert (got - ref[i]).abs().max() <= tiny.tolerance(dtype, ref[i]), f"position {i}"

    one_by_one(2030, 2070)                                      # across position 2,048
    runner.step([StepEntry("long", toks[2070:2290], [])])       # the gap as one portion
    one_by_one(2290, 2300)
    assert runner.steps == 1 + 6 + 40 + 1 + 10
    if dtype == "bfloat16":
        assert runner.graphs is not None and runner.graphs.replays >= 45, "the single tokens replay captured steps"
    runner.finish("long")
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_single_rows_beside_portions(name, dtype, built, plain_logits):
    """A mixed step: requests that bring one token beside portions of prompts. Where their rows lie together the
    bfloat16 attention takes them through the kernel for single rows (the step's description says so); where a
    portion stands between them they are tiles of one row. Either way every row matches the plain implementation."""
    from jllm_serve_amd.engine.step import StepEntry
    model, runner = built(name, dtype)
    a, b, c, p, q = (tiny.prompt(name, n, seed=20 + n) for n in (70, 33, 17, 150, 41))
    for rid in ("sa", "sb", "sc", "sp", "sq"):
        runner.finish(rid)
    runner.step([StepEntry("sa", a[:-1], []), StepEntry("sb", b[:-1], []), StepEntry("sc", c[:-1], [])])

    def check(out, parts):
        at = 0
        for tokens, first, n in parts:
            ref = plain_logits(name, tokens)[first:first + n]
            assert (out[at:at + n].cpu().double() - ref).abs().max() <= tiny.tolerance(dtype, ref)
            at += n
    described = []
    layout = runner._layout

    def watched(*args, **kw):  # what the attention's step planner said about the batch
        r = layout(*args, **kw)
        described.append({key[0]: facts for key, _, _, facts in r[1]["plans"]}["gqa"])
        return r
    runner._layout = watched
    try:
        together = [StepEntry("sp", p[:140], range(140)), StepEntry("sa", a[-1:], [0]), StepEntry("sb", b[-1:], [0])]
        check(runner.step(together), [(p, 0, 140), (a, len(a) - 1, 1), (b, len(b) - 1, 1)])
        assert described[-1]["single_rows"] == (140, 2) and described[-1]["n_tiles_multi"] == 2
        apart = [StepEntry("sc", c[-1:], [0]), StepEntry("sp", p[140:], range(10)), StepEntry("sa", [5], [0])]
        check(runner.step(apart), [(c, len(c) - 1, 1), (p, 140, 10), (a + [5], len(a), 1)])
        assert described[-1]["single_rows"] is None and described[-1]["n_tiles"] == 3
        runner.finish("sp")
        a_pair_and_two = [StepEntry("sq", q[:2], [1]), StepEntry("sb", [9], [0]), StepEntry("sc", [3], [0])]
        check(runner.step(a_pair_and_two), [(q, 1, 1), (b + [9], len(b), 1), (c + [3], len(c), 1)])
        assert described[-1]["single_rows"] == (2, 2)
    finally:
        runner._layout = layout
        for rid in ("sa", "sb", "sc", "sp", "sq"):
            runner.finish(rid)


def test_schedule_may_repeat_a_layer_and_share_a_cache(model_folders):
    """The order of layers is data: a schedule that runs layer 0 twice (two caches) and lets a third run read the
    cache of the first instead of writing one. Checked against the plain parts put together the same way."""
    from jllm_serve_amd.config import ScheduleEntry, load_config
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.engine import build_model, build_runner
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights import SafetensorsSource
    folder = model_folders["A"]
    base = load_config(folder)
    sched = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_from=1))
    cfg = ModelConfig(**{**base.__dict__, "schedule": sched})
    model = build_model(cfg, SafetensorsSource(folder), "float32", torch.device(DEV), 128)
    runner = build_runner(model, page_size=8, pool_tokens=128, max_requests=2)
    assert len(runner.cache.groups) == 1 and len(runner.cache.groups[0].runs) == 3
    toks = tiny.prompt("A", 21)
    got = torch.cat([runner.step([StepEntry("s", toks[:13], list(range(13)))]),
                     runner.step([StepEntry("s", toks[13:], list(range(8)))])]).cpu().double()
    # plain: run 3 uses layer 1's weights on its own input for q, but the keys and values that run 1 computed
    pc = P.read_config(tiny.TINY_A)
    w = tiny.load_weights(folder)
    x = P.embedding(w["model.embed_tokens.weight"], toks)
    pos = torch.arange(len(toks))
    kv_of_run1 = None
    for run, e in enumerate(sched):
        prefix = f"model.layers.{e.layer}"
        xb = P.rmsnorm(x, w[prefix + ".input_layernorm.weight"], pc["eps"])
        p = prefix + ".self_attn."
        T, H, Hkv, hd = len(toks), pc["heads"], pc["kv_heads"], pc["head_dim"]
        cos, sin = P.rope_angles(pos, pc["rotary_dim"], pc["theta"])
        q = P.apply_rope(P.rmsnorm(P.linear(xb, w[p + "q_proj.weight"]).view(T, H, hd), w[p + "q_norm.weight"], pc["eps"]), cos, sin)
        if e.cache_from is None:
            k = P.apply_rope(P.rmsnorm(P.linear(xb, w[p + "k_proj.weight"]).view(T, Hkv, hd), w[p + "k_norm.weight"], pc["eps"]), cos, sin)
            v = P.linear(xb, w[p + "v_proj.weight"]).view(T, Hkv, hd)
            if run == 1:
                kv_of_run1 = (k, v)
        else:
            k, v = kv_of_run1
        att = P.attention(q, k, v, 1 / math.sqrt(hd)).reshape(T, H * hd)
        x = x + P.linear(att, w[p + "o_proj.weight"])
        xb = P.rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], pc["eps"])
        m = prefix + ".mlp."
        x = x + P.swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])
    ref = P.linear(P.rmsnorm(x, w["model.norm.weight"], pc["eps"]), w["model.embed_tokens.weight"])
    assert (got - ref).abs().max() <= tiny.tolerance("float32", ref)


def test_checkpoint_stored_in_32_bit_runs_in_both_types(tmp_path, plain_logits):
    """A tensor stored in 32-bit stays 32-bit in a bfloat16 run (activations and cache are bfloat16 then, the
    products take mixed operands); a float32 run widens nothing. Both must agree with the plain model."""
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "f32"), tiny.TINY_B, seed=11, dtype=torch.float32)
    toks = tiny.prompt("B", 45, seed=6)
    ref = tiny.plain_forward(folder, toks)
    for dtype in ("float32", "bfloat16"):
        model = load_model(folder, dtype, torch.device(DEV), max_positions=128)
        assert model.embed.dtype == torch.float32 and model.layers[0].mixer.w_qkv.dtype == torch.float32
        runner = build_runner(model, page_size=16, pool_tokens=128, max_requests=2)
        assert runner.cache.groups[0].storage["k"].dtype == (torch.float32 if dtype == "float32" else torch.bfloat16)
        got = torch.cat([runner.step([StepEntry("r", toks[:31], list(range(31)))]),
                         runner.step([StepEntry("r", toks[31:44], list(range(13)))]),
                         runner.step([StepEntry("r", toks[44:], [0])])]).cpu().double()
        assert (got - ref).abs().max() <= tiny.tolerance(dtype, ref)
