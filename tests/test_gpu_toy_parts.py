"""Two more toy parts, defined here and registered without a change to the framework's files: a feed-forward that
routes every row to one of a few small experts, and a position encoding with its own table of angles. A toy
architecture puts them into some layers of a model whose other layers keep the dense feed-forward and the usual
rotary table, so one model has different feed-forwards and different position encodings in different layers.
Nothing here is anyone's model."""
import json
import os
from dataclasses import dataclass

import pytest
import torch

import tiny
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


@dataclass(frozen=True)
class RoutedSpec:
    experts: int
    hidden: int
    kind: str = "toy_routed"


@dataclass(frozen=True)
class StepAngleSpec:
    """Angles position * step * (pair + 1) over the first `rotary_dim` dims (a law of its own, not the geometric one)."""
    rotary_dim: int
    step: float
    kind: str = "toy_step_angles"


def make_routed():
    from jllm_serve_amd.kernels import ops
    from jllm_serve_amd.parts import Part
    from jllm_serve_amd.weights import WeightSpec

    class Routed(Part):
        """x += expert_e(xb) with e = argmax of a router product in 32-bit; experts are small gated feed-forwards.
        The routing (which rows go where) is host-visible torch indexing: this is a toy."""

        def __init__(self, spec, prefix, build):
            self.spec, self.prefix, self.build = spec, prefix, build
            self.router = None
            self.experts = []

        def names(self, e):
            p = f"{self.prefix}.toy_experts.{e}."
            return p + "gate.weight", p + "up.weight", p + "down.weight"

        def weight_specs(self):
            d, f = self.build.hidden, self.spec.hidden
            out = [WeightSpec(self.prefix + ".toy_router.weight", (self.spec.experts, d))]
            for e in range(self.spec.experts):
                g, u, dn = self.names(e)
                out += [WeightSpec(g, (f, d)), WeightSpec(u, (f, d)), WeightSpec(dn, (d, f))]
            return out

        def load(self, get):
            self.router = get(self.prefix + ".toy_router.weight")
            self.experts = [tuple(get(n) for n in self.names(e)) for e in range(self.spec.experts)]

        def forward(self, xb, residual, step):
            logits = ops.gemm(xb.float(), self.router.float(), out_dtype=torch.float32, exact=True)  # router in 32-bit
            choice = ops.argmax(logits)
            for e, (g, u, dn) in enumerate(self.experts):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel() == 0:
                    continue
                h = ops.gemm(xb[rows].contiguous(), g, w2=u, epilogue=ops.EPI_GATED, exact=self.build.exact)
                y = ops.gemm(h, dn, out_dtype=torch.float32, exact=self.build.exact)
                residual.index_add_(0, rows, y)
    return Routed


def make_step_angles():
    from jllm_serve_amd.parts import Part

    class StepAngles(Part):
        def __init__(self, spec, build):
            self.spec = spec
            pos = torch.arange(build.max_positions, dtype=torch.float64)[:, None]
            pair = torch.arange(1, spec.rotary_dim // 2 + 1, dtype=torch.float64)[None, :]
            ang = pos * spec.step * pair
            self.cos, self.sin = torch.cos(ang).float().to(build.device), torch.sin(ang).float().to(build.device)

        def rotary(self):
            return self.cos, self.sin, self.spec.rotary_dim
    return StepAngles


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_toy_positions(dtype, tmp_path):
    from dataclasses import replace
    from jllm_serve_amd.config import parse_config, register_architecture, unregister_architecture
    from jllm_serve_amd.config.schema import ModelConfig
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.parts import register_part, unregister_part
    from jllm_serve_amd.parts.model import DecoderModel
    from jllm_serve_amd.weights import RandomSource, write_safetensors

    base_cfg = {**tiny.TINY_D, "num_hidden_layers": 3}
    E, F_EXPERT, ROT, STEP = 3, 128, 64, 0.011

    def parse_toy(c, model_type, arch):
        base = parse_config(base_cfg)
        layers = list(base.layers)
        # layer 1: routed feed-forward; layer 2: attention that reads the second position table
        layers[1] = replace(layers[1], ffn=RoutedSpec(experts=E, hidden=F_EXPERT))
        layers[2] = replace(layers[2], mixer=replace(layers[2].mixer, position=len(base.positions)))
        return ModelConfig(**{**base.__dict__, "layers": tuple(layers),
                              "positions": tuple(base.positions) + (StepAngleSpec(rotary_dim=ROT, step=STEP),),
                              "model_type": model_type, "architecture": arch})

    register_part("ffn", "toy_routed", make_routed())
    register_part("position", "toy_step_angles", make_step_angles())
    register_architecture("toy_routed_model", "ToyRoutedForCausalLM", parse_toy)
    try:
        folder = str(tmp_path / "toy")
        os.makedirs(folder)
        cfg_d = {"model_type": "toy_routed_model", "architectures": ["ToyRoutedForCausalLM"]}
        json.dump(cfg_d, open(os.path.join(folder, "config.json"), "w"))
        cfg = parse_config(cfg_d)
        specs = DecoderModel(cfg, torch.float32, "cpu", 1).weight_specs()
        names = [s.name for s in specs]
        assert "model.layers.1.toy_router.weight" in names and not any(n.startswith("model.layers.1.mlp.") for n in names)
        assert any(n.startswith("model.layers.0.mlp.") for n in names)
        src = RandomSource(specs, seed=11, dtype=torch.bfloat16)
        tensors = {n: src.get(n) for n in src.names()}
        # a router that decides clearly (a bfloat16 run must route like the 32-bit one)
        tensors["model.layers.1.toy_router.weight"] = (tensors["model.layers.1.toy_router.weight"].float() * 40).bfloat16()
        write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
        model = load_model(folder, dtype, torch.device(DEV), max_positions=128)
        runner = build_runner(model, page_size=16, pool_tokens=256, max_requests=3, graphs=False)

        w = {n: t.double() for n, t in tensors.items()}
        pc = P.read_config(base_cfg)
        hd, H, Hkv = pc["head_dim"], pc["heads"], pc["kv_heads"]

        def attention_with_step_angles(xb, prefix, pos):
            """Plain attention of layer 2 with the toy angles: the same parts as the plain model, another table."""
            q = P.linear(xb, w[prefix + ".self_attn.q_proj.weight"]).view(-1, H, hd)
            k = P.linear(xb, w[prefix + ".self_attn.k_proj.weight"]).view(-1, Hkv, hd)
            v = P.linear(xb, w[prefix + ".self_attn.v_proj.weight"]).view(-1, Hkv, hd)
            q = P.rmsnorm(q, w[prefix + ".self_attn.q_norm.weight"], pc["eps"])
            k = P.rmsnorm(k, w[prefix + ".self_attn.k_norm.weight"], pc["eps"])
            ang = pos.double()[:, None] * STEP * torch.arange(1, ROT // 2 + 1, dtype=torch.float64)[None, :]
            c, s = torch.cos(ang).float().double()[:, None, :], torch.sin(ang).float().double()[:, None, :]

            def rot(x):
                a, b = x[..., :ROT // 2], x[..., ROT // 2:ROT]
                return torch.cat([a * c - b * s, b * c + a * s, x[..., ROT:]], -1)
            q, k = rot(q), rot(k)
            T = q.shape[0]
            out = torch.zeros(T, H, hd, dtype=torch.float64)
            for h in range(H):
                kk, vv = k[:, h // (H // Hkv)], v[:, h // (H // Hkv)]
                sc = (q[:, h] @ kk.T) / (hd ** 0.5)
                sc = sc.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
                out[:, h] = torch.softmax(sc, -1) @ vv
            return P.linear(out.reshape(T, H * hd), w[prefix + ".self_attn.o_proj.weight"])

        def plain(tokens):
            x = P.embedding(w["model.embed_tokens.weight"], tokens)
            pos = torch.arange(len(tokens))
            routes = None
            for l in range(3):
                prefix = f"model.layers.{l}"
                xb = P.rmsnorm(x, w[prefix + ".input_layernorm.weight"], pc["eps"])
                x = x + (attention_with_step_angles(xb, prefix, pos) if l == 2 else P.attention_block(xb, w, prefix, pc, l, pos))
                xb = P.rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], pc["eps"])
                if l == 1:
                    routes = torch.argmax(xb @ w[prefix + ".toy_router.weight"].T, -1)
                    y = torch.zeros_like(x)
                    for e in range(E):
                        p_ = f"{prefix}.toy_experts.{e}."
                        y[routes == e] = P.swiglu(xb[routes == e], w[p_ + "gate.weight"], w[p_ + "up.weight"], w[p_ + "down.weight"])
                    x = x + y
                else:
                    m = prefix + ".mlp."
                    x = x + P.swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])
            return P.linear(P.rmsnorm(x, w["model.norm.weight"], pc["eps"]), w["lm_head.weight"]), routes

        a, b = tiny.prompt("D", 45, seed=1), tiny.prompt("D", 30, seed=2)
        (ra, routes_a), (rb, _) = plain(a), plain(b)
        assert len(set(routes_a.tolist())) >= 2, "the prompt should reach more than one expert"
        got_a, got_b = [], []
        pa = pb = 0
        for na, nb in zip([20, 2, 1, 21, 1], [7, 1, 19, 2, 1]):  # portions beside single tokens, cut anywhere
            out = runner.step([StepEntry("a", a[pa:pa + na], range(na)), StepEntry("b", b[pb:pb + nb], range(nb))]).cpu().double()
            got_a.append(out[:na]); got_b.append(out[na:])
            pa += na; pb += nb
        assert pa == len(a) and pb == len(b)
        assert (torch.cat(got_a) - ra).abs().max() <= tiny.tolerance(dtype, ra)
        assert (torch.cat(got_b) - rb).abs().max() <= tiny.tolerance(dtype, rb)
    finally:
        unregister_part("ffn", "toy_routed")
        unregister_part("position", "toy_step_angles")
        unregister_architecture("toy_routed_model")
