"""config.json -> typed configuration; the registry; the reference's validation errors."""
import json

import pytest

import tiny
from jllm_serve_amd.config import (ConfigError, ScheduleEntry, load_config, parse_config, register_architecture,
                                   supported, unregister_architecture)
from jllm_serve_amd.config.schema import ModelConfig

Q8B = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=36, hidden_size=4096,
           num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
           rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960,
           sliding_window=None, use_sliding_window=False, max_window_layers=36, eos_token_id=151645, bos_token_id=151643)


def test_tiny_a_and_b_and_8b_parse():
    a = parse_config(tiny.TINY_A)
    assert (a.hidden, a.vocab, a.num_layers, a.tie_embeddings, a.max_positions) == (64, 256, 2, True, 128)
    m = a.layers[0].mixer
    assert (m.heads, m.kv_heads, m.head_dim, m.window, m.qk_norm, m.bias, m.out_bias) == (4, 2, 16, 0, True, False, False)
    assert a.positions[0].theta == 10000.0 and a.positions[0].rotary_dim == 16 and a.final_norm.eps == 1e-6
    assert m.scale == pytest.approx(0.25)
    b = parse_config(tiny.TINY_B)
    assert b.layers[2].mixer.q_dim == 192 != b.hidden and b.layers[0].mixer.group == 3
    assert b.positions[0].theta == 1e6 and b.final_norm.eps == 1e-5 and not b.tie_embeddings
    c = parse_config(Q8B)
    assert c.layers[35].ffn.hidden == 12288 and c.eos_token_ids == (151645,) and c.bos_token_id == 151643
    assert all(l.mixer.window == 0 for l in c.layers)
    assert c.description == ("Qwen3ForCausalLM dim=4096 ffn=12288 layers=36 heads=32/8 headDim=128 vocab=151936 theta=1000000")
    assert [e.layer for e in c.schedule] == list(range(36)) and all(e.cache_from is None for e in c.schedule)


def test_tiny_c_options():
    c = parse_config(tiny.TINY_C)
    assert [l.mixer.window for l in c.layers] == [0, 0, 20, 20]  # layers >= max_window_layers (Families.java:773-787)
    assert c.layers[0].mixer.bias and c.layers[0].mixer.out_bias  # attention_bias => q,k,v and o (Families.java:167)
    assert " bias obias" in c.description and "window=20@2" in c.description  # T/SmokeTest.java:848-856
    assert c.positions[0].scaling.kind == "yarn" and c.positions[0].scaling.original_max_positions == 64
    assert c.eos_token_ids == (7, 300) and c.layers[0].mixer.qk_norm_eps == 1e-4


def test_defaults():
    c = parse_config(dict(model_type="qwen3", hidden_size=32, num_hidden_layers=1, vocab_size=10,
                          num_attention_heads=4, intermediate_size=8))
    m = c.layers[0].mixer
    assert (m.kv_heads, m.head_dim) == (4, 8)  # Families.java:717-719
    assert c.positions[0].theta == 1e4 and c.final_norm.eps == 1e-6 and c.max_positions == 4096
    assert not c.tie_embeddings and c.bos_token_id == -1 and c.eos_token_ids == ()
    # sliding_window without use_sliding_window stays off
    c = parse_config({**tiny.TINY_A, "sliding_window": 8})
    assert all(l.mixer.window == 0 for l in c.layers)
    # rope_parameters (nested) is read when the top-level key is absent; the top-level key wins
    d = {k: v for k, v in tiny.TINY_A.items() if k != "rope_theta"}
    assert parse_config({**d, "rope_parameters": {"rope_theta": 777.0}}).positions[0].theta == 777.0
    assert parse_config({**tiny.TINY_A, "rope_parameters": {"rope_theta": 777.0}}).positions[0].theta == 10000.0
    assert parse_config({**tiny.TINY_A, "partial_rotary_factor": 0.5}).positions[0].rotary_dim == 8


def test_model_type_from_architectures_and_unknown():
    d = {k: v for k, v in tiny.TINY_A.items() if k != "model_type"}
    assert parse_config(d).model_type == "qwen3"
    with pytest.raises(ConfigError, match="unsupported model"):
        parse_config({**tiny.TINY_A, "model_type": "llama"})
    with pytest.raises(ConfigError, match="unsupported model"):
        parse_config({**tiny.TINY_A, "architectures": ["LlamaForCausalLM"]})
    assert supported()["qwen3"] == "Qwen3ForCausalLM"


@pytest.mark.parametrize("patch,msg", [
    ({"hidden_size": 0}, "hidden_size must be a positive integer"),
    ({"num_hidden_layers": -1}, "num_hidden_layers must be a positive integer"),
    ({"vocab_size": None}, "vocab_size must be a positive integer"),
    ({"num_key_value_heads": 3}, "must be positive and divide"),
    ({"num_key_value_heads": 0}, "must be positive and divide"),
    ({"head_dim": 0}, "head_dim must be positive"),
    ({"hidden_act": "gelu"}, "unsupported hidden_act 'gelu'"),
    ({"mlp_bias": True}, "MLP bias"),
    ({"partial_rotary_factor": 1.5}, "invalid partial_rotary_factor"),
    ({"intermediate_size": 0}, "intermediate_size must be positive"),
    ({"eos_token_id": "x"}, "must be an int or a list of ints"),
    ({"eos_token_id": [1, 2.5]}, "must be an int or a list of ints"),
    ({"rope_scaling": {"rope_type": "ntk", "factor": 2}}, "unsupported rope_scaling type 'ntk'"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 0}}, "invalid yarn"),
    ({"rope_scaling": {"rope_type": "linear", "factor": -1}}, "invalid linear"),
    ({"num_experts": 8}, "qwen3_moe"),
])
def test_validation_errors(patch, msg):
    with pytest.raises(ConfigError, match=msg):
        parse_config({**tiny.TINY_A, **patch})


def test_load_config_errors(tmp_path):
    with pytest.raises(ConfigError, match="no such file"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_B))
    assert load_config(str(tmp_path)).hidden == 96


def test_schedule_is_data_and_checked():
    a = parse_config(tiny.TINY_A)
    twice = ModelConfig(**{**a.__dict__, "schedule": (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_from=1))})
    assert len(twice.schedule) == 4
    with pytest.raises(ConfigError):
        ModelConfig(**{**a.__dict__, "schedule": (ScheduleEntry(0), ScheduleEntry(5))})
    with pytest.raises(ConfigError):
        ModelConfig(**{**a.__dict__, "schedule": (ScheduleEntry(0, cache_from=0),)})


def test_another_architecture_can_be_registered():
    def parse(c, model_type, arch):
        base = parse_config({**tiny.TINY_A, "num_hidden_layers": c["depth"]})
        return ModelConfig(**{**base.__dict__, "model_type": model_type, "architecture": arch})
    register_architecture("toy_arch", "ToyForCausalLM", parse)
    try:
        cfg = parse_config({"model_type": "toy_arch", "depth": 5})
        assert cfg.num_layers == 5 and cfg.architecture == "ToyForCausalLM"
        with pytest.raises(ValueError):
            register_architecture("toy_arch", "ToyForCausalLM", parse)
    finally:
        unregister_architecture("toy_arch")
