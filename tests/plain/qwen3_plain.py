"""A plain, slow Qwen3-dense forward pass: whole sequences, no cache, one function per part.

Written from the reference's formulas (every docstring gives file:line under src/main/java/org/robomiri/jllm/ of the
reference's tree); it shares no code with the engine. Everything is torch on the CPU in the dtype of its inputs
(tests use float64). The config is the raw config.json dict, read here independently of the engine's parser.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------------------- config


def read_config(c: dict) -> dict:
    """The keys the Qwen3 family reads and their defaults (model/Families.java:710-733, :735-800, :166-171)."""
    heads = c["num_attention_heads"]
    dim = c["hidden_size"]
    layers = c["num_hidden_layers"]
    window = 0
    window_from = 0
    if (c.get("sliding_window") or 0) > 0 and c.get("use_sliding_window", False):  # :773-787
        window = c["sliding_window"]
        window_from = c.get("max_window_layers", layers)
    head_dim = c.get("head_dim", dim // heads)
    return dict(dim=dim, layers=layers, vocab=c["vocab_size"], heads=heads,
                kv_heads=c.get("num_key_value_heads", heads), head_dim=head_dim,
                ffn=c["intermediate_size"], eps=c.get("rms_norm_eps", 1e-6), theta=c.get("rope_theta", 1e4),
                rotary_dim=int(head_dim * c.get("partial_rotary_factor", 1.0)) & ~1,
                rope_scaling=c.get("rope_scaling"), max_pos=c.get("max_position_embeddings", 4096),
                bias=c.get("attention_bias", False), tied=c.get("tie_word_embeddings", False),
                window=window, window_from=window_from)


# ----------------------------------------------------------------------------------------------- parts


def embedding(table: torch.Tensor, ids: List[int]) -> torch.Tensor:
    """x[t, :] = E[token[t], :]; embedScale is 1 for Qwen3 (cpu/CpuBackend.java:947-958; model/Families.java:678)."""
    return table[torch.tensor(ids, dtype=torch.long)]


def rmsnorm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """out[i] = (x[i] * (1 / sqrt(sum(x^2)/n + eps))) * g[i] over the last dim (cpu/VectorKernels.java:630-634)."""
    ss = (x * x).sum(dim=-1, keepdim=True)
    scale = 1.0 / torch.sqrt(ss / x.shape[-1] + eps)
    return (x * scale) * g


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, r] = sum_c W[r, c] * x[t, c] (+ b[r]), W is [out, in] (cpu/CpuMatmul.java:8-31; bias
    cpu/CpuBackend.java:430-436)."""
    y = torch.einsum("tc,rc->tr", x, w)
    return y if b is None else y + b


def rope_inv_freq(rotary_dim: int, theta: float, scaling: Optional[dict], max_pos: int) -> torch.Tensor:
    """model/Rope.java:122-167 (plain, linear, llama3) and :190-208 (yarn), in float64."""
    half = rotary_dim // 2
    i = torch.arange(half, dtype=torch.float64)
    f = 1.0 / torch.pow(torch.tensor(float(theta), dtype=torch.float64), (2.0 * i) / rotary_dim)
    kind = "default" if not scaling else scaling.get("rope_type", scaling.get("type", "default"))
    if kind in ("default", "mrope"):
        return f
    factor = float(scaling.get("factor", 1.0))
    if kind == "linear":
        return f / factor
    if kind == "llama3":
        low, high = scaling.get("low_freq_factor", 1.0), scaling.get("high_freq_factor", 4.0)
        orig = scaling.get("original_max_position_embeddings", 8192)
        out = f.clone()
        for k in range(half):
            wavelen = 2 * math.pi / f[k].item()
            if wavelen < orig / high:
                continue
            if wavelen > orig / low:
                out[k] = f[k] / factor
            else:
                smooth = (orig / wavelen - low) / (high - low) if high - low > 0 else 0.0
                out[k] = (1 - smooth) * f[k] / factor + smooth * f[k]
        return out
    if kind == "yarn":
        orig = scaling.get("original_max_position_embeddings", max_pos)
        beta_fast, beta_slow = scaling.get("beta_fast", 32), scaling.get("beta_slow", 1)
        truncate = scaling.get("truncate", True)

        def corr(rot):  # yarnCorrectionDim, model/Rope.java:176-178
            return rotary_dim * math.log(orig / (rot * 2 * math.pi)) / (2 * math.log(theta))
        lo, hi = corr(beta_fast), corr(beta_slow)
        low = max(math.floor(lo) if truncate else lo, 0)
        high = min(math.ceil(hi) if truncate else hi, rotary_dim - 1)
        if low == high:
            high += 0.001
        ramp = torch.clamp((i - low) / (high - low), 0, 1)
        return (f / factor) * ramp + f * (1 - ramp)
    raise ValueError(kind)


def rope_amplitude(scaling: Optional[dict]) -> float:
    """model/Rope.java:75-85: YaRN's attention_factor, else mscale ratio, else 0.1 ln(factor) + 1; 1 otherwise."""
    if not scaling or scaling.get("rope_type", scaling.get("type")) != "yarn":
        return 1.0
    if scaling.get("attention_factor", 0) > 0:
        return float(scaling["attention_factor"])
    factor = float(scaling.get("factor", 1.0))
    ms, msa = scaling.get("mscale", 0), scaling.get("mscale_all_dim", 0)
    both = ms != 0 and msa != 0
    ms, msa = (ms, msa) if both else (1.0, 0.0)

    def yarn_mscale(scale, m):  # model/Rope.java:170-172
        return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0
    return yarn_mscale(factor, ms) / yarn_mscale(factor, msa)


def rope_angles(positions: torch.Tensor, rotary_dim: int, theta: float, scaling=None, max_pos: int = 4096):
    """cos/sin [len(positions), rotary_dim/2]: angle p * invFreq[i] in double, rounded to float32 as the
    reference's table is (model/Rope.java:24-38)."""
    inv = rope_inv_freq(rotary_dim, theta, scaling, max_pos)
    amp = rope_amplitude(scaling)
    ang = positions.to(torch.float64)[:, None] * inv[None, :]
    return (torch.cos(ang) * amp).to(torch.float32), (torch.sin(ang) * amp).to(torch.float32)


def apply_rope(v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """v [T, heads, hd]; rotate-half pairing over the first 2*half dims: (a, b) = (v[i], v[i+half]) ->
    (a cos - b sin, b cos + a sin) (cpu/VectorKernels.java:692-711); dims beyond the rotary width stay."""
    half = cos.shape[-1]
    c = cos.to(v.dtype)[:, None, :]
    s = sin.to(v.dtype)[:, None, :]
    a, b = v[..., :half], v[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., 2 * half:]], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int = 0,
              pos0: int = 0) -> torch.Tensor:
    """q [T, H, hd], k/v [T, Hkv, hd] of one whole sequence starting at position pos0. Query head h uses kv
    head h // G; s_j = (q . k_j) * scale; the row at position p sees keys j in [max(0, p + 1 - window), p]
    (window 0: from 0) (model/Attention.java:68-71); softmax with max-subtract, then the weighted sum of v
    (cpu/KvCache.java:455-464, :1034-1071)."""
    T, H, hd = q.shape
    Hkv = k.shape[1]
    G = H // Hkv
    out = torch.zeros_like(q)
    for h in range(H):
        kh, vh = k[:, h // G, :], v[:, h // G, :]
        for t in range(T):
            first = max(0, (pos0 + t) + 1 - window) - pos0 if window > 0 else 0
            first = max(first, 0)
            s = (kh[first:t + 1] @ q[t, h]) * scale
            e = torch.exp(s - s.max())
            p = e * (1.0 / e.sum())
            out[t, h] = p @ vh[first:t + 1]
    return out


def silu(z: torch.Tensor) -> torch.Tensor:
    """z / (1 + exp(-z)) (cpu/VectorKernels.java:637-639)."""
    return z / (1.0 + torch.exp(-z))


def swiglu(xb: torch.Tensor, w_gate, w_up, w_down) -> torch.Tensor:
    """W_down (silu(W_gate xb) * (W_up xb)) (cpu/CpuBackend.java:661-669, :1289-1300)."""
    return linear(silu(linear(xb, w_gate)) * linear(xb, w_up), w_down)


def attention_block(xb, w: Dict[str, torch.Tensor], prefix: str, cfg: dict, layer: int, positions: torch.Tensor):
    """Projections (+ biases), per-head q/k RMSNorm with shared gains BEFORE the rotation, rotation of q and k
    (v untouched), causal GQA, output projection (cpu/CpuBackend.java:423-457, :595-633)."""
    p = prefix + ".self_attn."
    T = xb.shape[0]
    H, Hkv, hd = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    b = (lambda n: w[p + n + "_proj.bias"]) if cfg["bias"] else (lambda n: None)
    q = linear(xb, w[p + "q_proj.weight"], b("q")).view(T, H, hd)
    k = linear(xb, w[p + "k_proj.weight"], b("k")).view(T, Hkv, hd)
    v = linear(xb, w[p + "v_proj.weight"], b("v")).view(T, Hkv, hd)
    q = rmsnorm(q, w[p + "q_norm.weight"], cfg["eps"])
    k = rmsnorm(k, w[p + "k_norm.weight"], cfg["eps"])
    cos, sin = rope_angles(positions, cfg["rotary_dim"], cfg["theta"], cfg["rope_scaling"], cfg["max_pos"])
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    window = cfg["window"] if cfg["window"] > 0 and layer >= cfg["window_from"] else 0
    scale = float(torch.tensor(1.0 / math.sqrt(hd), dtype=torch.float32))  # (float)(1/sqrt(hd)), model/Families.java:861
    att = attention(q, k, v, scale, window, int(positions[0])).reshape(T, H * hd)
    return linear(att, w[p + "o_proj.weight"], w.get(p + "o_proj.bias") if cfg["bias"] else None)


def decoder_layer(x, w, layer: int, cfg: dict, positions):
    """xb = rmsnorm(x; g_in); x += attn(xb); xb = rmsnorm(x; g_post); x += mlp(xb) (cpu/CpuBackend.java:959-969)."""
    prefix = f"model.layers.{layer}"
    xb = rmsnorm(x, w[prefix + ".input_layernorm.weight"], cfg["eps"])
    x = x + attention_block(xb, w, prefix, cfg, layer, positions)
    xb = rmsnorm(x, w[prefix + ".post_attention_layernorm.weight"], cfg["eps"])
    m = prefix + ".mlp."
    return x + swiglu(xb, w[m + "gate_proj.weight"], w[m + "up_proj.weight"], w[m + "down_proj.weight"])


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64) -> torch.Tensor:
    """Logits [len(tokens), vocab] of one whole sequence from position 0: embedding, L layers, final norm, output
    head = lm_head.weight when present else the embedding (model/ModelWeights.java:36-43; cpu/CpuBackend.java:980-985)."""
    cfg = read_config(config)
    w = {k: v.to(dtype) for k, v in weights.items()}
    x = embedding(w["model.embed_tokens.weight"], tokens)
    positions = torch.arange(len(tokens))
    for l in range(cfg["layers"]):
        x = decoder_layer(x, w, l, cfg, positions)
    xb = rmsnorm(x, w["model.norm.weight"], cfg["eps"])
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(xb, head)


def greedy(config: dict, weights, prompt: List[int], n: int, dtype=torch.float64) -> List[int]:
    """Greedy continuation by recomputing the whole sequence for every token; argmax = lowest index among
    equal maxima (sampling/Sampler.java:458-466)."""
    toks = list(prompt)
    out = []
    for _ in range(n):
        z = forward(config, weights, toks, dtype)[-1]
        t = int(torch.argmax(z))  # torch returns the first maximum
        out.append(t)
        toks.append(t)
    return out
