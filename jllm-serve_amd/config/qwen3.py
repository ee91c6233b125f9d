"""The Qwen3 dense family: config.json keys -> ModelConfig.

What the reference's parser does for ``model_type: "qwen3"`` (model/Families.java:162-171 sets the
family switches; the shared Draft reads the keys, :710-733, and builds the layer specs, :735-916):

* required positive ints ``hidden_size``, ``num_hidden_layers``, ``vocab_size``, ``num_attention_heads``;
  ``num_key_value_heads`` defaults to the head count, ``head_dim`` to hidden/heads (:714-720);
* per-head q/k RMSNorm is on (:168); biases only with ``attention_bias`` and then on q, k, v and o_proj (:167);
* the window rule of Qwen2: ``sliding_window`` applies to layers >= ``max_window_layers`` and only when
  ``use_sliding_window`` is true (:169, :773-787);
* ``rope_theta`` (default 1e4) and ``partial_rotary_factor`` also from a nested ``rope_parameters``,
  the top-level key wins (:721-732, :766-772); scaling from ``rope_scaling`` (:1001-1072);
* ``hidden_act`` must be silu, ``mlp_bias`` is refused (:743-751); ``num_experts`` > 0 is the MoE family,
  which this engine does not build.
"""
from __future__ import annotations

import math
from typing import Any, Mapping, Optional, Tuple

from .registry import register_architecture
from .schema import (ConfigError, GatedMlpNames, GatedMlpSpec, GqaNames, GqaSpec, LayerSpec, ModelConfig, ModelNames,
                     NormSpec, RopeScaling, RopeSpec, default_schedule)


def _num(c: Optional[Mapping[str, Any]], key: str, default):
    """json/Json.java:421-424: a number, else the default (null and other types fall back too)."""
    v = c.get(key) if isinstance(c, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        return default
    return v


def _int(c, key, default: int) -> int:
    return int(_num(c, key, default))


def _bool(c, key: str, default: bool) -> bool:
    v = c.get(key) if isinstance(c, Mapping) else None
    return v if isinstance(v, bool) else default


def _str(c, key: str, default):
    v = c.get(key) if isinstance(c, Mapping) else None
    return v if isinstance(v, str) else default


def _map(c, key: str):
    v = c.get(key) if isinstance(c, Mapping) else None
    return v if isinstance(v, Mapping) else None


def require_positive(c: Mapping[str, Any], key: str) -> int:
    """model/Families.java:1126-1133."""
    v = _num(c, key, 0)
    if v != int(v) or int(v) <= 0 or int(v) > 2**31 - 1:
        got = c[key] if key in c else "nothing"
        raise ConfigError(f"config.json: {key} must be a positive integer, got {got}")
    return int(v)


def int_list(c: Mapping[str, Any], key: str) -> Tuple[int, ...]:
    """model/Families.java:1099-1118: absent/null -> (), an int -> one entry, a list of ints; else an error."""
    v = c.get(key)
    if v is None:
        return ()
    if isinstance(v, bool):
        raise ConfigError(f"config.json: {key} must be an int or a list of ints, got {v}")
    if isinstance(v, (int, float)):
        return (int(v),)
    if isinstance(v, (list, tuple)):
        out = []
        for o in v:
            if isinstance(o, bool) or not isinstance(o, (int, float)) or float(o) != int(o):
                raise ConfigError(f"config.json: {key} must be an int or a list of ints, got {v}")
            out.append(int(o))
        return tuple(out)
    raise ConfigError(f"config.json: {key} must be an int or a list of ints, got {v}")


def parse_rope_scaling(rs: Optional[Mapping[str, Any]], c: Mapping[str, Any]) -> RopeScaling:
    """model/Families.java:1001-1072. ``longrope`` is read by the reference for other families; Qwen3
    checkpoints use none or yarn, so it is refused here with the list of what is built."""
    if rs is None:
        return RopeScaling()
    kind = _str(rs, "rope_type", _str(rs, "type", "default"))
    factor = float(_num(rs, "factor", 1.0))
    if kind in ("default", "mrope"):
        return RopeScaling()
    if kind == "linear":
        if factor <= 0:
            raise ConfigError(f"invalid linear rope_scaling: {dict(rs)}")
        return RopeScaling(kind="linear", factor=factor)
    if kind == "llama3":
        low = float(_num(rs, "low_freq_factor", 1.0))
        high = float(_num(rs, "high_freq_factor", 4.0))
        orig = _int(rs, "original_max_position_embeddings", 8192)
        if factor <= 0 or low <= 0 or high < low or orig <= 0:
            raise ConfigError(f"invalid llama3 rope_scaling: {dict(rs)}")
        return RopeScaling(kind="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
                           original_max_positions=orig)
    if kind == "yarn":
        orig = _int(rs, "original_max_position_embeddings", _int(c, "max_position_embeddings", 0))
        beta_fast = float(_num(rs, "beta_fast", 32))
        beta_slow = float(_num(rs, "beta_slow", 1))
        attention = float(_num(rs, "attention_factor", 0))
        if not factor > 0 or orig <= 0 or not beta_fast > beta_slow or not beta_slow > 0 or attention < 0:
            raise ConfigError(f"invalid yarn rope_scaling: {dict(rs)}")
        mscale = float(_num(rs, "mscale", 0))
        mscale_all = float(_num(rs, "mscale_all_dim", 0))
        both = mscale != 0 and mscale_all != 0
        return RopeScaling(kind="yarn", factor=factor, original_max_positions=orig, beta_fast=beta_fast,
                           beta_slow=beta_slow, mscale=mscale if both else 1.0,
                           mscale_all_dim=mscale_all if both else 0.0, attention_factor=attention,
                           truncate=_bool(rs, "truncate", True))
    raise ConfigError(f"unsupported rope_scaling type '{kind}' (supported: default, linear, llama3, yarn)")


def parse_qwen3(c: Mapping[str, Any], model_type: str, architecture: str) -> ModelConfig:
    dim = require_positive(c, "hidden_size")
    n_layers = require_positive(c, "num_hidden_layers")
    vocab = require_positive(c, "vocab_size")
    heads = require_positive(c, "num_attention_heads")
    kv_heads = _int(c, "num_key_value_heads", heads)
    head_dim = _int(c, "head_dim", dim // heads)
    ffn = _int(c, "intermediate_size", 0)

    rope_params = _map(c, "rope_parameters")
    full_rope = _map(rope_params, "full_attention")
    global_rope = full_rope if full_rope is not None else rope_params
    rs = _map(c, "rope_scaling")
    if rs is None and global_rope is not None and ("rope_type" in global_rope or "type" in global_rope):
        rs = global_rope

    if kv_heads <= 0 or heads % kv_heads != 0:
        raise ConfigError(f"num_key_value_heads={kv_heads} must be positive and divide num_attention_heads={heads}")
    if head_dim <= 0:
        raise ConfigError(f"head_dim must be positive, got {head_dim}")
    act = _str(c, "hidden_act", "silu")
    if act != "silu":
        raise ConfigError(f"unsupported hidden_act '{act}': only silu (SwiGLU) is implemented")
    if _bool(c, "mlp_bias", False):
        raise ConfigError("models with an MLP bias (mlp_bias=true) are not supported")
    attn_bias = _bool(c, "attention_bias", False)
    partial = float(_num(c, "partial_rotary_factor", _num(global_rope, "partial_rotary_factor", 1.0)))
    if partial <= 0 or partial > 1 or int(head_dim * partial) < 2:
        raise ConfigError(f"invalid partial_rotary_factor {partial}")
    rotary_dim = int(head_dim * partial) & ~1
    theta = float(_num(c, "rope_theta", _num(global_rope, "rope_theta", 1e4)))
    window = 0
    window_from = 0
    sw_raw = _int(c, "sliding_window", 0)
    if sw_raw > 0 and _bool(c, "use_sliding_window", False):
        window = min(sw_raw, 2**31 - 1)
        window_from = _int(c, "max_window_layers", n_layers)
    scaling = parse_rope_scaling(rs, c)
    eos = int_list(c, "eos_token_id")
    eps = float(_num(c, "rms_norm_eps", 1e-6))
    if _int(c, "num_experts", 0) > 0:
        raise ConfigError("num_experts > 0 is the qwen3_moe family; this engine builds Qwen3 dense only")
    if ffn <= 0:
        raise ConfigError("intermediate_size must be positive for a model with dense MLP layers")

    rope = RopeSpec(rotary_dim=rotary_dim, theta=theta, scaling=scaling, pairing="half")
    scale = float(1.0 / math.sqrt(head_dim))  # model/Families.java:861
    norm = NormSpec(eps=eps)
    # the checkpoint's tensor names (model/AttnWeights.java:20-45, model/MlpWeights.java:19-33, model/ModelWeights.java:36-43)
    attn_names = GqaNames(q="self_attn.q_proj", k="self_attn.k_proj", v="self_attn.v_proj", o="self_attn.o_proj",
                          q_norm="self_attn.q_norm", k_norm="self_attn.k_norm")
    mlp_names = GatedMlpNames(gate="mlp.gate_proj", up="mlp.up_proj", down="mlp.down_proj")
    layers = []
    for l in range(n_layers):
        windowed = window > 0 and l >= window_from
        mixer = GqaSpec(heads=heads, kv_heads=kv_heads, head_dim=head_dim, scale=scale,
                        window=window if windowed else 0, position=0, qk_norm=True, qk_norm_eps=eps,
                        bias=attn_bias, out_bias=attn_bias, names=attn_names)
        layers.append(LayerSpec(mixer=mixer, ffn=GatedMlpSpec(hidden=ffn, activation="silu", names=mlp_names), norm=norm,
                                prefix=f"model.layers.{l}", norm_in_name="input_layernorm",
                                norm_post_name="post_attention_layernorm"))

    # the canonical one-line description (model/Families.java:887-910), with the parts Qwen3 can set
    extra = (" bias obias" if attn_bias else "")
    if window > 0:
        extra += f" window={window}" + (f"@{window_from}" if window_from > 0 else "")
    if scaling.kind != "none":
        extra += f" rope={scaling.kind}x{scaling.factor}"
    if rotary_dim != head_dim:
        extra += f" rotary={rotary_dim}"
    description = (f"{architecture} dim={dim} ffn={ffn} layers={n_layers} heads={heads}/{kv_heads} "
                   f"headDim={head_dim} vocab={vocab} theta={theta:.0f}{extra}")
    return ModelConfig(
        architecture=architecture, model_type=model_type, hidden=dim, vocab=vocab, final_norm=norm,
        layers=tuple(layers), positions=(rope,), schedule=default_schedule(n_layers),
        tie_embeddings=_bool(c, "tie_word_embeddings", False), bos_token_id=_int(c, "bos_token_id", -1),
        eos_token_ids=eos, max_positions=_int(c, "max_position_embeddings", 4096), embed_scale=1.0,
        description=description,
        names=ModelNames(embed="model.embed_tokens.weight", final_norm="model.norm.weight", head="lm_head.weight"),
        raw=dict(c))


register_architecture("qwen3", "Qwen3ForCausalLM", parse_qwen3, replace=True)
