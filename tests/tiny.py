"""The tiny configurations the tests run, and helpers shared by them.

A and B are the two tiny Qwen3-dense configurations of the benchmark description; C adds the options the
other two leave off (window on the upper layers, q/k/v/o biases, YaRN scaling, one kv head per query head,
a head size that is no power of two, an odd vocabulary). Between them every size and option differs.
"""
import json
import os
import random

import torch

TINY_A = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=64,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, vocab_size=256,
              rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=128)
TINY_B = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=3, hidden_size=96,
              num_attention_heads=6, num_key_value_heads=2, head_dim=32, intermediate_size=224, vocab_size=384,
              rope_theta=1e6, rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=256)
TINY_C = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=4, hidden_size=80,
              num_attention_heads=5, num_key_value_heads=5, head_dim=48, intermediate_size=176, vocab_size=301,
              rope_theta=5e5, rms_norm_eps=1e-4, tie_word_embeddings=False, max_position_embeddings=192,
              attention_bias=True, use_sliding_window=True, sliding_window=20, max_window_layers=2,
              rope_scaling={"rope_type": "yarn", "factor": 2.0, "original_max_position_embeddings": 64},
              eos_token_id=[7, 300], bos_token_id=1)

# sizes the matrix-core kernels take (K multiples of 128, head size 128), so the bfloat16 run goes through them
TINY_D = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=256,
              num_attention_heads=4, num_key_value_heads=2, head_dim=128, intermediate_size=384, vocab_size=512,
              rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=512)

# the proportions of the smallest released checkpoint (hidden 1024, 16 query heads over 8 key heads of 128, tied
# embeddings) with three layers and an odd vocabulary of a realistic width; pages of 64
SMALL_E = dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=3, hidden_size=1024,
               num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=32003,
               rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=1024)

# name -> (config, weight seed, page size)
CONFIGS = {"A": (TINY_A, 0, 8), "B": (TINY_B, 1, 16), "C": (TINY_C, 2, 32), "D": (TINY_D, 3, 16), "E": (SMALL_E, 4, 64)}


def prompt(name: str, length: int, seed: int = 0):
    rng = random.Random(f"{name}/{length}/{seed}")
    v = CONFIGS[name][0]["vocab_size"]
    return [rng.randrange(v) for _ in range(length)]


def load_weights(folder: str, dtype=torch.float64):
    """Reads the folder with the safetensors *format* package (not the engine's reader)."""
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k).to(dtype)
    return out


def plain_forward(folder: str, tokens):
    from plain import qwen3_plain
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return qwen3_plain.forward(cfg, load_weights(folder), list(tokens))


def tolerance(dtype: str, ref: torch.Tensor):
    """fp32: the reference's own bound for equal passes (MixedPassChecks.java:237-243: 1e-4 of the largest logit
    + 1e-5). bf16: 1.5 % of the largest logit."""
    m = float(ref.abs().max())
    return 1e-4 * m + 1e-5 if dtype == "float32" else 1.5e-2 * m
