"""A toy mixer with state of its own, defined here, registered, built and stepped without a change to the
framework's files: a running mean of the inputs per request, kept in a fixed-size state slot. It is registered
beside a toy architecture whose layers alternate it with attention, so one model has different mixers in
different layers. Nothing here is anyone's model."""
from dataclasses import dataclass

import pytest
import torch

import tiny
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


@dataclass(frozen=True)
class RunningMeanSpec:
    width: int
    kind: str = "toy_running_mean"


def make_part():
    from jllm_serve_amd.cache import StateSpec
    from jllm_serve_amd.parts import Part
    from jllm_serve_amd.weights import WeightSpec

    class RunningMean(Part):
        """y_t = W (mean of xb_0..xb_t): needs the sum of all earlier inputs and their count, nothing per position."""
        capturable = False  # walks the step's requests on the host

        def __init__(self, spec, prefix, build, positions):
            self.spec, self.prefix, self.build = spec, prefix, build
            self.w = None

        def weight_specs(self):
            return [WeightSpec(self.prefix + ".toy.weight", (self.build.hidden, self.spec.width))]

        def load(self, get):
            self.w = get(self.prefix + ".toy.weight")

        def state_spec(self):
            return StateSpec((self.spec.width + 1,), torch.float32)  # running sum and count

        def forward(self, xb, residual, step, slot):
            for seg in step.segments:  # a request's rows are contiguous and in order
                st = slot.state[seg.state_slot]
                rows = xb[seg.row0:seg.row0 + seg.n].float()
                sums = st[:-1] + torch.cumsum(rows, 0)
                counts = st[-1] + torch.arange(1, seg.n + 1, device=rows.device, dtype=torch.float32)
                residual[seg.row0:seg.row0 + seg.n] += (sums / counts[:, None]) @ self.w.float().T
                st[:-1] = sums[-1]
                st[-1] = counts[-1]
    return RunningMean


def test_toy_mixer_with_state(model_folders, tmp_path):
    from jllm_serve_amd.config import parse_config, register_architecture, unregister_architecture
    from jllm_serve_amd.config.schema import LayerSpec, ModelConfig
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.parts import register_part, unregister_part
    from jllm_serve_amd.weights import RandomSource, write_safetensors
    from jllm_serve_amd.parts.model import DecoderModel
    import json, os

    def parse_toy(c, model_type, arch):
        base = parse_config({**tiny.TINY_B, "num_hidden_layers": 3})
        layers = list(base.layers)
        layers[1] = LayerSpec(mixer=RunningMeanSpec(width=base.hidden), ffn=base.layers[1].ffn, norm=base.layers[1].norm,
                              prefix=base.layers[1].prefix)
        return ModelConfig(**{**base.__dict__, "layers": tuple(layers), "model_type": model_type, "architecture": arch})

    register_part("mixer", "toy_running_mean", make_part())
    register_architecture("toy_mean", "ToyMeanForCausalLM", parse_toy)
    try:
        folder = str(tmp_path / "toy")
        os.makedirs(folder)
        cfg_d = {"model_type": "toy_mean", "architectures": ["ToyMeanForCausalLM"]}
        json.dump(cfg_d, open(os.path.join(folder, "config.json"), "w"))
        cfg = parse_config(cfg_d)
        specs = DecoderModel(cfg, torch.float32, "cpu", 1).weight_specs()
        assert any(s.name.endswith(".toy.weight") for s in specs) and not any("layers.1.self_attn" in s.name for s in specs)
        src = RandomSource(specs, seed=3, dtype=torch.float32)
        write_safetensors(os.path.join(folder, "model.safetensors"), {n: src.get(n) for n in src.names()})
        model = load_model(folder, "float32", torch.device(DEV), max_positions=128)  # through the registry, by config.json
        runner = build_runner(model, page_size=16, pool_tokens=256, max_requests=3)
        # layers 0 and 2 own pages (one group, two runs), layer 1 owns a state slot and no pages
        assert len(runner.cache.groups) == 1 and runner.cache.groups[0].runs == [0, 2]
        assert runner.cache.slots[1].state is not None and runner.cache.slots[1].group is None

        w = {n: src.get(n).double() for n in src.names()}
        pc = P.read_config({**tiny.TINY_B, "num_hidden_layers": 3})

        def plain(tokens):
            x = P.embedding(w["model.embed_tokens.weight"], tokens)
            pos = torch.arange(len(tokens))
            for l in range(3):
                prefix = f"model.layers.{l}"
                xb = P.rmsnorm(x, w[prefix + ".input_layernorm.weight"], pc["eps"])
                if l == 1:
                    mean = torch.cumsum(xb, 0) / torch.arange(1, len(tokens) + 1, dtype=torch.float64)[:, None]
                    x = x + mean @ w[prefix + ".toy.weight"].T
                else:
                    x = x + P.attention_block(xb, w, prefix, pc, l, pos)
                xb = P.rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], pc["eps"])
                m = prefix + ".mlp."
                x = x + P.swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])
            return P.linear(P.rmsnorm(x, w["model.norm.weight"], pc["eps"]), w["lm_head.weight"])

        a, b = tiny.prompt("B", 40, seed=1), tiny.prompt("B", 23, seed=2)
        ra, rb = plain(a), plain(b)
        # two requests stepped in portions beside each other, then token by token; a third reuses a's slot afterwards
        got_a, got_b = [], []
        cuts_a, cuts_b = [9, 2, 17, 1, 1, 10], [5, 11, 2, 3, 1, 1]
        pa = pb = 0
        for na, nb in zip(cuts_a, cuts_b):
            out = runner.step([StepEntry("a", a[pa:pa + na], range(na)), StepEntry("b", b[pb:pb + nb], range(nb))]).cpu().double()
            got_a.append(out[:na]); got_b.append(out[na:])
            pa += na; pb += nb
        assert pa == len(a) and pb == len(b)
        assert (torch.cat(got_a) - ra).abs().max() <= tiny.tolerance("float32", ra)
        assert (torch.cat(got_b) - rb).abs().max() <= tiny.tolerance("float32", rb)
        runner.finish("a")
        c = tiny.prompt("B", 12, seed=3)
        out = runner.step([StepEntry("c", c, range(len(c)))]).cpu().double()
        assert (out - plain(c)).abs().max() <= tiny.tolerance("float32", plain(c)), "a reused state slot starts from zero"
        with pytest.raises(ValueError, match="cannot be rewound"):
            runner.cache.truncate("c", 3)
    finally:
        unregister_part("mixer", "toy_running_mean")
        unregister_architecture("toy_mean")
