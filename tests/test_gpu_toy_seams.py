"""Three more toys, each defined here and registered without a change to the framework's files, one for each seam
that another architecture would come in through:

* a mixer that keeps ONE tensor per position in pages (not a key and a value) and brings its own per-step metadata
  (a step planner: for every row the list of cache slots it reads);
* a position encoding that rotates nothing: it adds a learned table to the embedded rows and a distance bias to
  the attention scores, and has tensors of its own;
* a checkpoint with other tensor names and stacked projections (one qkv tensor, one gate/up tensor): only the
  parser's name tables change.

Nothing here is anyone's model."""
import json
import os
from dataclasses import dataclass, replace

import numpy as np
import pytest
import torch

import tiny
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ------------------------------------------------------------------------------------------------ one tensor per position


@dataclass(frozen=True)
class WindowMeanSpec:
    """y_t = W_o mean(c_j for j in the last `window` positions up to t), c_j = W_c xb_j kept in pages."""
    width: int
    window: int
    kind: str = "toy_window_mean"


def make_window_mean():
    from jllm_serve_amd.cache import CacheRow, PageSpec
    from jllm_serve_amd.engine.step import StepPlan
    from jllm_serve_amd.parts import Part
    from jllm_serve_amd.weights import WeightSpec

    class ReadListPlanner:
        """For every row of the step: the cache slots (page * page size + offset) of the positions it reads, flattened,
        and which row each belongs to. Built from the block tables on the host; rides in the step's one upload."""

        def __init__(self, page_spec):
            self.page_spec = page_spec
            self.key = ("toy_window_mean", page_spec)

        def plan(self, batch):
            gi = batch.cache.group_index(self.page_spec)
            B, w = batch.page_size, self.page_spec.window
            slots, owner = [], []
            for s in batch.segments:
                table = batch.cache.table(s.rid, gi)
                for i in range(s.n):
                    p = s.pos0 + i
                    for j in range(max(0, p + 1 - w), p + 1):
                        assert table[j // B] >= 0, "a position inside the window lies in a page that was given back"
                        slots.append(table[j // B] * B + j % B)
                        owner.append(s.row0 + i)
            return StepPlan({"slots": slots, "owner": owner}, {"reads": len(slots)})

    class WindowMean(Part):
        capturable = False  # its plan's arrays grow with the contexts: not a step of fixed size

        def __init__(self, spec, prefix, build, positions):
            self.spec, self.prefix, self.build = spec, prefix, build
            self.wc = self.wo = None

        def weight_specs(self):
            return [WeightSpec(self.prefix + ".toy.c.weight", (self.spec.width, self.build.hidden)),
                    WeightSpec(self.prefix + ".toy.o.weight", (self.build.hidden, self.spec.width))]

        def load(self, get):
            self.wc, self.wo = get(self.prefix + ".toy.c.weight"), get(self.prefix + ".toy.o.weight")

        def cache_spec(self):
            return PageSpec((CacheRow("c", (self.spec.width,), 0, torch.float32),), self.spec.window)

        def step_planners(self):
            return [ReadListPlanner(self.cache_spec())]

        def forward(self, xb, residual, step, slot):
            plan = step.plans[("toy_window_mean", self.cache_spec())]
            cache = slot.rows["c"].view(-1, self.spec.width)  # [pages * page size, width]
            c = xb.float() @ self.wc.float().T
            cache[step.groups[slot.group].slots.long()] = c  # store first, as the kernels do
            got = cache[plan.arrays["slots"].long()]
            owner = plan.arrays["owner"].long()
            sums = torch.zeros_like(c).index_add_(0, owner, got)
            counts = torch.zeros(c.shape[0], device=c.device).index_add_(0, owner, torch.ones_like(owner, dtype=torch.float32))
            residual += (sums / counts[:, None]) @ self.wo.float().T
    return WindowMean


def test_toy_mixer_with_one_cached_tensor_and_its_own_step_plan(tmp_path):
    from jllm_serve_amd.config import parse_config, register_architecture, unregister_architecture
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.parts import register_part, unregister_part
    from jllm_serve_amd.parts.model import DecoderModel
    from jllm_serve_amd.weights import RandomSource, write_safetensors
    WIDTH, WINDOW, PAGE = 24, 20, 8

    def parse_toy(c, model_type, arch):
        base = parse_config({**tiny.TINY_B, "num_hidden_layers": 3})
        layers = list(base.layers)
        layers[1] = replace(layers[1], mixer=WindowMeanSpec(width=WIDTH, window=WINDOW))
        return ModelConfig(**{**base.__dict__, "layers": tuple(layers), "model_type": model_type, "architecture": arch})

    register_part("mixer", "toy_window_mean", make_window_mean())
    register_architecture("toy_window", "ToyWindowForCausalLM", parse_toy)
    try:
        folder = str(tmp_path / "toy")
        os.makedirs(folder)
        cfg_d = {"model_type": "toy_window", "architectures": ["ToyWindowForCausalLM"]}
        json.dump(cfg_d, open(os.path.join(folder, "config.json"), "w"))
        cfg = parse_config(cfg_d)
        specs = DecoderModel(cfg, torch.float32, "cpu", 1).weight_specs()
        src = RandomSource(specs, seed=5, dtype=torch.float32)
        write_safetensors(os.path.join(folder, "model.safetensors"), {n: src.get(n) for n in src.names()})
        model = load_model(folder, "float32", torch.device(DEV), max_positions=128)
        runner = build_runner(model, page_size=PAGE, pool_tokens=20 * PAGE, max_requests=3)
        # two groups: attention's (layers 0 and 2: a key and a value per position) and the toy's (one tensor, a window)
        assert [(g.runs, sorted(g.storage), g.spec.window) for g in runner.cache.groups] == [([0, 2], ["k", "v"], 0), ([1], ["c"], WINDOW)]
        assert runner.cache.groups[1].storage["c"].shape == (1, 20, PAGE, WIDTH)
        assert [pl.key[0] for pl in runner.planners()] == ["gqa", "toy_window_mean"], "two attention layers plan once"

        w = {n: src.get(n).double() for n in src.names()}
        pc = P.read_config({**tiny.TINY_B, "num_hidden_layers": 3})

        def plain(tokens):
            x = P.embedding(w["model.embed_tokens.weight"], tokens)
            pos = torch.arange(len(tokens))
            for l in range(3):
                prefix = f"model.layers.{l}"
                xb = P.rmsnorm(x, w[prefix + ".input_layernorm.weight"], pc["eps"])
                if l == 1:
                    c = xb @ w[prefix + ".toy.c.weight"].T
                    mean = torch.stack([c[max(0, t + 1 - WINDOW):t + 1].mean(0) for t in range(len(tokens))])
                    x = x + mean @ w[prefix + ".toy.o.weight"].T
                else:
                    x = x + P.attention_block(xb, w, prefix, pc, l, pos)
                xb = P.rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], pc["eps"])
                m = prefix + ".mlp."
                x = x + P.swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])
            return P.linear(P.rmsnorm(x, w["model.norm.weight"], pc["eps"]), w["lm_head.weight"])

        a, b = tiny.prompt("B", 61, seed=1), tiny.prompt("B", 37, seed=2)
        ra, rb = plain(a), plain(b)
        got_a, got_b = [], []
        pa = pb = 0
        for na, nb in zip([9, 2, 30, 1, 1, 18], [5, 11, 2, 17, 1, 1]):  # portions beside single tokens, cut anywhere
            out = runner.step([StepEntry("a", a[pa:pa + na], range(na)), StepEntry("b", b[pb:pb + nb], range(nb))]).cpu().double()
            got_a.append(out[:na]); got_b.append(out[na:])
            pa += na; pb += nb
            runner.cache.check()
        assert pa == len(a) and pb == len(b)
        assert (torch.cat(got_a) - ra).abs().max() <= tiny.tolerance("float32", ra)
        assert (torch.cat(got_b) - rb).abs().max() <= tiny.tolerance("float32", rb)
        assert runner.cache.pages_given_back_by_window > 0, "the toy's window gives pages back while attention keeps all"
        held = [sum(1 for p in runner.cache.table("a", gi) if p >= 0) for gi in range(2)]
        assert held == [8, 3], held  # 61 positions: 8 pages of keys and values; the last 20 touch 3 pages of the toy's
        runner.finish("a")
        runner.finish("b")
        assert all(g.pool.used_pages == 0 for g in runner.cache.groups)
        c_ = tiny.prompt("B", 12, seed=3)  # pages that the toy used before, used again
        out = runner.step([StepEntry("c", c_, range(len(c_)))]).cpu().double()
        assert (out - plain(c_)).abs().max() <= tiny.tolerance("float32", plain(c_))
    finally:
        unregister_part("mixer", "toy_window_mean")
        unregister_architecture("toy_window")


# ------------------------------------------------------------------------------------------------ a position encoding that rotates nothing


@dataclass(frozen=True)
class AddedAndBiasedSpec:
    """A learned table added to the embedded rows, and a bias slope * (key position - query position) on the scores."""
    rows: int
    slope: float
    kind: str = "toy_added_and_biased"


def make_added_and_biased():
    from jllm_serve_amd.parts import Part
    from jllm_serve_amd.weights import WeightSpec

    class AddedAndBiased(Part):
        def __init__(self, spec, build):
            self.spec, self.build = spec, build
            self.table = None

        def weight_specs(self):
            return [WeightSpec("toy_positions.weight", (self.spec.rows, self.build.hidden))]

        def load(self, get):
            self.table = get("toy_positions.weight")

        def rotary(self):
            return None  # q and k are not rotated

        def embed_add(self, x, step):
            x += self.table[step.positions.long()].float()

        def score_bias(self, heads):
            return (torch.arange(1, heads + 1, dtype=torch.float32, device=self.build.device) * self.spec.slope).contiguous()
    return AddedAndBiased


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_added_at_the_input_and_as_a_score_bias(dtype, tmp_path):
    from jllm_serve_amd.config import parse_config, register_architecture, unregister_architecture
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.parts import register_part, unregister_part
    from jllm_serve_amd.parts.model import DecoderModel
    from jllm_serve_amd.weights import RandomSource, write_safetensors
    SLOPE, ROWS = 0.07, 96
    base_cfg = {**tiny.TINY_B, "num_hidden_layers": 2}

    def parse_toy(c, model_type, arch):
        base = parse_config(base_cfg)
        layers = [replace(l, mixer=replace(l.mixer, position=0)) for l in base.layers]
        return ModelConfig(**{**base.__dict__, "layers": tuple(layers), "positions": (AddedAndBiasedSpec(ROWS, SLOPE),),
                              "model_type": model_type, "architecture": arch})

    register_part("position", "toy_added_and_biased", make_added_and_biased())
    register_architecture("toy_biased", "ToyBiasedForCausalLM", parse_toy)
    try:
        folder = str(tmp_path / "toy")
        os.makedirs(folder)
        cfg_d = {"model_type": "toy_biased", "architectures": ["ToyBiasedForCausalLM"]}
        json.dump(cfg_d, open(os.path.join(folder, "config.json"), "w"))
        cfg = parse_config(cfg_d)
        specs = DecoderModel(cfg, torch.float32, "cpu", 1).weight_specs()
        assert "toy_positions.weight" in [s.name for s in specs]
        src = RandomSource(specs, seed=9, dtype=torch.bfloat16)
        tensors = {n: src.get(n) for n in src.names()}
        write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
        model = load_model(folder, dtype, torch.device(DEV), max_positions=ROWS)
        runner = build_runner(model, page_size=16, pool_tokens=256, max_requests=2, graphs=False)
        w = {n: t.double() for n, t in tensors.items()}
        pc = P.read_config(base_cfg)
        H, Hkv, hd = pc["heads"], pc["kv_heads"], pc["head_dim"]

        def biased_attention(xb, prefix):
            T = xb.shape[0]
            q = P.rmsnorm(P.linear(xb, w[prefix + ".self_attn.q_proj.weight"]).view(T, H, hd), w[prefix + ".self_attn.q_norm.weight"], pc["eps"])
            k = P.rmsnorm(P.linear(xb, w[prefix + ".self_attn.k_proj.weight"]).view(T, Hkv, hd), w[prefix + ".self_attn.k_norm.weight"], pc["eps"])
            v = P.linear(xb, w[prefix + ".self_attn.v_proj.weight"]).view(T, Hkv, hd)
            dist = (torch.arange(T)[None, :] - torch.arange(T)[:, None]).double()  # key position - query position
            out = torch.zeros(T, H, hd, dtype=torch.float64)
            for h in range(H):
                sc = (q[:, h] @ k[:, h // (H // Hkv)].T) * float(np.float32(1.0 / np.sqrt(hd))) + SLOPE * (h + 1) * dist
                sc = sc.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
                out[:, h] = torch.softmax(sc, -1) @ v[:, h // (H // Hkv)]
            return P.linear(out.reshape(T, H * hd), w[prefix + ".self_attn.o_proj.weight"])

        def plain(tokens):
            x = P.embedding(w["model.embed_tokens.weight"], tokens) + w["toy_positions.weight"][:len(tokens)]
            for l in range(2):
                prefix = f"model.layers.{l}"
                x = x + biased_attention(P.rmsnorm(x, w[prefix + ".input_layernorm.weight"], pc["eps"]), prefix)
                xb = P.rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], pc["eps"])
                m = prefix + ".mlp."
                x = x + P.swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])
            return P.linear(P.rmsnorm(x, w["model.norm.weight"], pc["eps"]), w["lm_head.weight"])

        a = tiny.prompt("B", 50, seed=4)
        ra = plain(a)
        assert (ra - P.forward(base_cfg, {k_: v_ for k_, v_ in w.items() if k_ != "toy_positions.weight"}, a)).abs().max() > 1e-2, \
            "the toy encoding must matter"
        got, pa = [], 0
        for n in [17, 2, 1, 29, 1]:
            got.append(runner.step([StepEntry("a", a[pa:pa + n], range(n))]).cpu().double())
            pa += n
        assert (torch.cat(got) - ra).abs().max() <= tiny.tolerance(dtype, ra)
    finally:
        unregister_part("position", "toy_added_and_biased")
        unregister_architecture("toy_biased")


# ------------------------------------------------------------------------------------------------ other names, stacked tensors


def test_a_checkpoint_with_other_names_and_stacked_projections_is_a_parser_change(model_folders, tmp_path):
    from jllm_serve_amd.config import (GatedMlpNames, GqaNames, ModelNames, parse_config, register_architecture,
                                       unregister_architecture)
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights import WeightError, write_safetensors

    def parse_renamed(c, model_type, arch):
        base = parse_config({**tiny.TINY_C, "model_type": "qwen3"})
        layers = []
        for i, l in enumerate(base.layers):
            mixer = replace(l.mixer, names=GqaNames(qkv="attn.wqkv", o="attn.wo", q_norm="attn.qn", k_norm="attn.kn"))
            ffn = replace(l.ffn, names=GatedMlpNames(gate_up="ffn.w13", down="ffn.w2"))
            layers.append(replace(l, mixer=mixer, ffn=ffn, prefix=f"blocks.{i}", norm_in_name="ln1", norm_post_name="ln2"))
        return ModelConfig(**{**base.__dict__, "layers": tuple(layers), "model_type": model_type, "architecture": arch,
                              "names": ModelNames(embed="tok.weight", final_norm="ln_f.weight", head="out.weight")})

    register_architecture("toy_renamed", "ToyRenamedForCausalLM", parse_renamed)
    try:
        std = tiny.load_weights(model_folders["C"], torch.bfloat16)
        new = {"tok.weight": std["model.embed_tokens.weight"], "ln_f.weight": std["model.norm.weight"], "out.weight": std["lm_head.weight"]}
        for i in range(tiny.TINY_C["num_hidden_layers"]):
            a, b = f"model.layers.{i}.", f"blocks.{i}."
            new[b + "attn.wqkv.weight"] = torch.cat([std[a + f"self_attn.{n}_proj.weight"] for n in "qkv"])
            new[b + "attn.wqkv.bias"] = torch.cat([std[a + f"self_attn.{n}_proj.bias"] for n in "qkv"])
            new[b + "attn.wo.weight"], new[b + "attn.wo.bias"] = std[a + "self_attn.o_proj.weight"], std[a + "self_attn.o_proj.bias"]
            new[b + "attn.qn.weight"], new[b + "attn.kn.weight"] = std[a + "self_attn.q_norm.weight"], std[a + "self_attn.k_norm.weight"]
            new[b + "ffn.w13.weight"] = torch.cat([std[a + "mlp.gate_proj.weight"], std[a + "mlp.up_proj.weight"]])
            new[b + "ffn.w2.weight"] = std[a + "mlp.down_proj.weight"]
            new[b + "ln1.weight"], new[b + "ln2.weight"] = std[a + "input_layernorm.weight"], std[a + "post_attention_layernorm.weight"]
        folder = str(tmp_path / "renamed")
        os.makedirs(folder)
        json.dump({"model_type": "toy_renamed", "architectures": ["ToyRenamedForCausalLM"]}, open(os.path.join(folder, "config.json"), "w"))
        write_safetensors(os.path.join(folder, "model.safetensors"), new)
        toks = tiny.prompt("C", 70)
        outs = []
        for d in (model_folders["C"], folder):
            runner = build_runner(load_model(d, "float32", torch.device(DEV), max_positions=192), page_size=32, pool_tokens=128,
                                  max_requests=1)
            outs.append(runner.step([StepEntry("r", toks, range(len(toks)))]))
        assert torch.equal(outs[0], outs[1]), "the same numbers under other names give the same logits, bit for bit"
        # and the load error speaks the checkpoint's language
        del new["blocks.2.ffn.w13.weight"]
        write_safetensors(os.path.join(folder, "model.safetensors"), new)
        with pytest.raises(WeightError, match=r"blocks\.2\.ffn\.w13\.weight"):
            load_model(folder, "float32", torch.device(DEV), max_positions=192)
    finally:
        unregister_architecture("toy_renamed")


# ------------------------------------------------------------------------------------------------ a model class of its own


def test_an_architecture_with_a_model_class_of_its_own_through_the_command_line(tmp_path, capsys):
    """An architecture registered with a model factory: its model wraps the generic decoder and has one tensor more
    (a bias added to the logits). The random-weights mode asks the registry's model class for the tensor list, so
    ``jllm random`` writes that tensor too and ``jllm run`` loads and runs the folder; the generated tokens are those of
    the plain implementation with the bias added. Registered here, no framework file changed."""
    from jllm_serve_amd.__main__ import main
    from jllm_serve_amd.config import parse_config, register_architecture, unregister_architecture
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.parts.model import DecoderModel
    from jllm_serve_amd.weights import WeightSpec

    def parse(c, model_type, arch):
        base = parse_config({**c, "model_type": "qwen3", "architectures": ["Qwen3ForCausalLM"]})
        return ModelConfig(**{**base.__dict__, "model_type": model_type, "architecture": arch})

    class BiasedHeadModel:
        """What a model factory returns: weight_specs / load / cache_plans / step_planners / forward, and the facts the
        runner reads (config, dtype, device, build, capturable)."""

        def __init__(self, config, dtype, device, max_positions):
            self.inner = DecoderModel(config, dtype, device, max_positions)
            self.config, self.dtype, self.device, self.build = config, self.inner.dtype, self.inner.device, self.inner.build
            self.capturable = self.inner.capturable
            self.bias = None

        def weight_specs(self):
            return self.inner.weight_specs() + [WeightSpec("toy.logit_bias", (self.config.vocab,), init="bias")]

        def load(self, source):
            from jllm_serve_amd.weights import check, fetch
            check(self.weight_specs(), source, where=self.config.description)
            names = [n for n in source.names() if n != "toy.logit_bias"]

            class Without:  # the inner model checks its own list: it must not see the extra tensor
                def names(self_):
                    return names

                def shape(self_, n):
                    return source.shape(n)

                def get(self_, n):
                    return source.get(n)
            self.inner.load(Without())
            self.bias = fetch(source, "toy.logit_bias", self.dtype, self.device).float()

        def cache_plans(self):
            return self.inner.cache_plans()

        def step_planners(self):
            return self.inner.step_planners()

        def forward(self, step, slots):
            return self.inner.forward(step, slots) + self.bias

    cfg_d = {**tiny.TINY_B, "model_type": "toy_biased_head", "architectures": ["ToyBiasedHeadForCausalLM"]}
    register_architecture("toy_biased_head", "ToyBiasedHeadForCausalLM", parse, model_factory=BiasedHeadModel)
    try:
        cfg_file = tmp_path / "toy.json"
        cfg_file.write_text(json.dumps(cfg_d))
        folder = str(tmp_path / "toy_model")
        assert main(["random", "--config-json", str(cfg_file), "--out", folder, "--seed", "3"]) == 0
        capsys.readouterr()
        w = tiny.load_weights(folder)
        assert "toy.logit_bias" in w and w["toy.logit_bias"].shape == (cfg_d["vocab_size"],)
        w["toy.logit_bias"] = w["toy.logit_bias"] * 40  # large enough to decide some tokens: written back below
        from jllm_serve_amd.weights import write_safetensors
        write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in w.items()})
        w = tiny.load_weights(folder)
        prompt = tiny.prompt("B", 11, seed=8)
        toks, want, plain_only = list(prompt), [], []
        inner = {k: v for k, v in w.items() if k != "toy.logit_bias"}
        for _ in range(6):
            z = P.forward(tiny.TINY_B, inner, toks)[-1]
            plain_only.append(int(torch.argmax(z)))
            want.append(int(torch.argmax(z + w["toy.logit_bias"])))
            toks.append(want[-1])
        assert want != plain_only, "the bias must decide at least one token, or the test shows nothing"
        rc = main(["run", "--model", folder, "--dtype", "float32", "--prompt", " ".join(map(str, prompt)), "--temp", "0",
                   "--max-tokens", "6", "--page-size", "16", "--ctx", "128", "--json"])
        out = capsys.readouterr()
        assert rc == 0, out.err
        assert json.loads(out.out.strip().splitlines()[-1])["tokens"] == want
    finally:
        unregister_architecture("toy_biased_head")
