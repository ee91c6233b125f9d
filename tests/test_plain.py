"""Pins the plain implementation by what fixes it beside the reference's text: vectors the reference's docs and
tests hold, special cases that reduce to a library routine, and invariants; each chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place) fails it. Also checks the engine's host-side rotary
tables against the same vectors."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import tiny
from plain import qwen3_plain as P
from jllm_serve_amd.config.schema import RopeScaling, RopeSpec
from jllm_serve_amd.parts import rope as engine_rope

D = torch.float64


def t(x):
    return torch.tensor(x, dtype=D)


def test_rmsnorm_vector_and_library():
    # docs/05-transformer-math.md:283-290
    y = P.rmsnorm(t([2, -4, 4, 2]), t([1, 1, 2, 1]), 0.0)
    assert torch.allclose(y, t([0.632, -1.265, 2.530, 0.632]), atol=1e-3)
    x = torch.randn(5, 24, dtype=D)
    g = torch.rand(24, dtype=D) + 0.5
    assert torch.allclose(P.rmsnorm(x, g, 1e-5), F.rms_norm(x, (24,), g, 1e-5), atol=1e-12)
    ones = torch.ones(24, dtype=D)
    assert torch.allclose((P.rmsnorm(x, ones, 0.0) ** 2).mean(-1), torch.ones(5, dtype=D))  # unit RMS
    assert torch.allclose(P.rmsnorm(3.7 * x, g, 0.0), P.rmsnorm(x, g, 0.0))  # scale invariant at eps 0
    assert torch.equal(P.rmsnorm(torch.zeros(4, dtype=D), torch.ones(4, dtype=D), 1e-6), torch.zeros(4, dtype=D))
    assert not torch.allclose(P.rmsnorm(x, g, 1e-5), F.layer_norm(x, (24,), g, None, 1e-5), atol=1e-3)  # no mean subtraction


def test_projection_vectors():
    # docs/05-transformer-math.md:370-383: W is [out, in]
    xb = t([[1.0, -0.5, 2.0]])
    assert torch.allclose(P.linear(xb, t([[0.5, 0, 1], [-1, 2, 0]])), t([[2.5, -2.0]]))
    assert torch.allclose(P.linear(xb, t([[1, 1, 0], [0, 0, 1]])), t([[0.5, 2.0]]))
    assert torch.allclose(P.linear(xb, t([[0, 1, 0], [1, 0, 0]])), t([[-0.5, 1.0]]))
    x, w, b = torch.randn(4, 7, dtype=D), torch.randn(5, 7, dtype=D), torch.randn(5, dtype=D)
    assert torch.allclose(P.linear(x, w, b), F.linear(x, w, b))


def test_embedding_and_output_head_vectors():
    E = t([[0.2, -1.0, 0.5], [0.9, 0.1, -0.3], [0.8, 0.2, -0.2], [-0.7, 0.6, 0.9]])  # docs/05:246-258
    assert torch.equal(P.embedding(E, [3, 0]), E[[3, 0]])
    logits = P.linear(t([[0.8, 0.3, -0.4]]), E)  # docs/05:892-903
    assert torch.allclose(logits, t([[-0.34, 0.87, 0.78, -0.74]]), atol=1e-9)


def test_silu_and_swiglu_vectors():
    assert torch.allclose(P.silu(t([-4, -1, 0, 1, 4])), t([-0.07, -0.27, 0, 0.73, 3.93]), atol=5e-3)  # docs/05:730-733
    z = torch.randn(50, dtype=D) * 3
    assert torch.allclose(P.silu(z), F.silu(z), atol=1e-12)
    out = P.swiglu(t([[1.0, 2.0]]), t([[1, 0], [-0.5, 0.5], [-1, -1]]), t([[0, 1], [1, 1], [2, 1.5]]),
                   t([[1, 0, 1], [0, 0.5, -1]]))  # docs/05:749-768
    assert torch.allclose(out, t([[0.751, 1.178]]), atol=2e-3)


def test_rope_frequencies_and_vectors():
    f = P.rope_inv_freq(128, 1e6, None, 4096)  # docs/05:468-476
    for i, v in ((0, 1.0), (16, 0.0316), (32, 0.001), (63, 1.2e-6)):
        assert f[i].item() == pytest.approx(v, rel=0.05)
    # key at 2, query at 5, theta = 1 (pair 0 of any table): score cos 3 = -0.990; same after a shift by 10 (docs/05:509-524)
    def score(p, s):
        cq, sq = P.rope_angles(torch.tensor([p]), 2, 1e4)
        ck, sk = P.rope_angles(torch.tensor([s]), 2, 1e4)
        q = P.apply_rope(t([[[1.0, 0.0]]]), cq, sq)
        k = P.apply_rope(t([[[1.0, 0.0]]]), ck, sk)
        return float((q * k).sum())
    assert score(5, 2) == pytest.approx(math.cos(3), abs=1e-6) == pytest.approx(-0.990, abs=1e-3)
    assert score(15, 12) == pytest.approx(score(5, 2), abs=1e-6)
    # the sign: rotating (1, 0) by the angle of position p gives (cos p, sin p), not (cos p, -sin p)
    c, s = P.rope_angles(torch.tensor([2]), 2, 1e4)
    assert torch.allclose(P.apply_rope(t([[[1.0, 0.0]]]), c, s).flatten(), t([math.cos(2), math.sin(2)]), atol=1e-6)


def test_rope_pairing_and_invariants():
    hd = 16
    pos = torch.tensor([0, 3, 11])
    cos, sin = P.rope_angles(pos, hd, 1e4)
    v = torch.randn(3, 2, hd, dtype=D)
    r = P.apply_rope(v, cos, sin)
    assert torch.allclose(r[0], v[0])  # position 0 is the identity
    assert torch.allclose(r.norm(dim=-1), v.norm(dim=-1), atol=1e-6)  # a rotation
    # a one-hot at index i moves only to i and i + hd/2 (rotate-half, not interleaved pairing)
    e = torch.zeros(1, 1, hd, dtype=D)
    e[0, 0, 3] = 1
    out = P.apply_rope(e, cos[1:2], sin[1:2]).flatten()
    assert set(torch.nonzero(out.abs() > 1e-12).flatten().tolist()) == {3, 3 + hd // 2}
    # the same through complex numbers: (v[i] + i v[i+half]) * exp(i p theta_i)
    inv = P.rope_inv_freq(hd, 1e4, None, 0)
    z = torch.complex(v[..., :hd // 2], v[..., hd // 2:]) * torch.exp(1j * (pos.to(D)[:, None] * inv[None, :]))[:, None, :]
    assert torch.allclose(torch.cat([z.real, z.imag], -1), r, atol=1e-6)
    # partial rotation leaves the dims beyond rotary_dim alone
    c8, s8 = P.rope_angles(pos, 8, 1e4)
    assert torch.equal(P.apply_rope(v, c8, s8)[..., 8:], v[..., 8:])
    # scores depend on the distance only
    q, k = torch.randn(1, 1, hd, dtype=D), torch.randn(1, 1, hd, dtype=D)
    def dot(p, s):
        cp, sp = P.rope_angles(torch.tensor([p]), hd, 1e4)
        cs, ss = P.rope_angles(torch.tensor([s]), hd, 1e4)
        return float((P.apply_rope(q, cp, sp) * P.apply_rope(k, cs, ss)).sum())
    assert dot(9, 4) == pytest.approx(dot(59, 54), abs=1e-5)


def test_rope_scaling_vectors():
    # T/SmokeTest.java:1498-1509 (yarn), :636-660 (llama3)
    y = {"rope_type": "yarn", "factor": 40, "original_max_position_embeddings": 4096}
    f = P.rope_inv_freq(64, 1e4, y, 4096)
    assert f[0] == 1.0 and abs(f[5] - 1e4 ** (-5 / 32)) < 1e-15 and abs(f[10] - 0.056234132519034905) < 1e-15
    assert abs(f[16] - 0.0055) < 1e-15 and abs(f[22] - 0.0001778279410038922) < 1e-15
    assert abs(f[23] - 3.33380358040831e-05) < 1e-18 and abs(f[31] - 1e4 ** (-31 / 32) / 40) < 1e-18
    assert P.rope_amplitude({"rope_type": "yarn", "factor": 4.0}) == pytest.approx(0.1 * math.log(4) + 1, abs=1e-15)
    assert P.rope_amplitude({**y, "mscale": 1.0, "mscale_all_dim": 0.707}) == pytest.approx(1.3688879454113936 / 1.2608037774058554)
    assert P.rope_amplitude({**y, "attention_factor": 1.5}) == 1.5
    l3 = {"rope_type": "llama3", "factor": 8, "low_freq_factor": 1, "high_freq_factor": 4, "original_max_position_embeddings": 8192}
    g = P.rope_inv_freq(8, 1e4, l3, 0)
    assert g[0] == 1.0 and abs(g[1] - 0.1) < 1e-15 and abs(g[3] - 2.1360754402756864e-4) < 1e-12
    h = P.rope_inv_freq(64, 5e5, l3, 0)
    assert abs(h[31] - 3.7673226901739635e-7) < 1e-18 and abs(h[1] - 0.6636012376960885) < 1e-12
    assert torch.allclose(P.rope_inv_freq(8, 1e4, {"type": "linear", "factor": 4}, 0), t([1, 0.1, 0.01, 0.001]) / 4)


def test_engine_rope_tables_hold_the_same_vectors():
    """The engine's table builder is separate code from the plain one; both must give the reference's numbers."""
    f = engine_rope.inverse_frequencies(RopeSpec(64, 1e4, RopeScaling(kind="yarn", factor=40, original_max_positions=4096)))
    assert f[0] == 1.0 and abs(f[16] - 0.0055) < 1e-15 and abs(f[22] - 0.0001778279410038922) < 1e-15
    l3 = RopeScaling(kind="llama3", factor=8, low_freq_factor=1, high_freq_factor=4, original_max_positions=8192)
    assert abs(engine_rope.inverse_frequencies(RopeSpec(8, 1e4, l3))[3] - 2.1360754402756864e-4) < 1e-12
    spec = RopeSpec(128, 1e6, RopeScaling(kind="yarn", factor=4.0, original_max_positions=32768))
    cos, sin = engine_rope.rope_table(spec, 3)
    amp = 0.1 * math.log(4) + 1
    inv = engine_rope.inverse_frequencies(spec)
    assert abs(cos[0, 0] - amp) < 1e-6 and abs(sin[2, 63] - math.sin(2 * inv[63]) * amp) < 1e-6  # T/SmokeTest.java:1540-1545
    for name in "ABC":
        cfg = P.read_config(tiny.CONFIGS[name][0])
        pc, ps = P.rope_angles(torch.arange(50), cfg["rotary_dim"], cfg["theta"], cfg["rope_scaling"], cfg["max_pos"])
        from jllm_serve_amd.config import parse_config
        ec, es = engine_rope.rope_table(parse_config(tiny.CONFIGS[name][0]).positions[0], 50)
        assert np.array_equal(pc.numpy(), ec) and np.array_equal(ps.numpy(), es)


def test_attention_vector_and_library():
    # docs/05-transformer-math.md:578-588
    q = t([[[0, 0]], [[0, 0]], [[1, 1]]])
    k = t([[[1, 0]], [[0, 1]], [[2, 2]]])
    v = t([[[1, 0]], [[0, 1]], [[5, 5]]])
    out = P.attention(q, k, v, 1 / math.sqrt(2))
    assert torch.allclose(out[2, 0], t([4.13, 4.13]), atol=5e-3)
    # no rotation, whole prompt: scaled_dot_product_attention with K/V repeated G times
    T, H, Hkv, hd = 9, 6, 2, 8
    q, k, v = torch.randn(T, H, hd, dtype=D), torch.randn(T, Hkv, hd, dtype=D), torch.randn(T, Hkv, hd, dtype=D)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(3, 1).transpose(0, 1),
                                         v.repeat_interleave(3, 1).transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(P.attention(q, k, v, 1 / math.sqrt(hd)), ref, atol=1e-12)
    assert torch.allclose(P.attention(q[:1], k[:1], v[:1], 0.3)[0, 4], v[0, 1])  # one visible key: output = its v; head 4 -> kv head 1
    # equal scores: the mean of v
    assert torch.allclose(P.attention(torch.zeros(T, H, hd, dtype=D), k, v, 1.0)[4, 0], v[:5, 0].mean(0))
    # later tokens never change an earlier row
    k2, v2 = k.clone(), v.clone()
    k2[6:] += 1; v2[6:] -= 2
    assert torch.equal(P.attention(q, k2, v2, 0.2)[:6], P.attention(q, k, v, 0.2)[:6])
    # window w: the row at p sees exactly keys p+1-w .. p (Attention.java:68-71)
    masked = torch.full((T, T), float("-inf"), dtype=D)
    for p in range(T):
        masked[p, max(0, p + 1 - 4):p + 1] = 0
    refw = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(3, 1).transpose(0, 1),
                                          v.repeat_interleave(3, 1).transpose(0, 1), attn_mask=masked).transpose(0, 1)
    assert torch.allclose(P.attention(q, k, v, 1 / math.sqrt(hd), window=4), refw, atol=1e-12)
    assert not torch.allclose(P.attention(q, k, v, 1 / math.sqrt(hd), window=4), ref, atol=1e-3)


def test_whole_model_closed_form_and_norm_order(model_folders):
    """Zero W_o and W_down: the residual passes through, logits = W_lm rmsnorm(E[id]) for any depth (docs/05:684-693)."""
    for name in "AB":
        cfg = tiny.CONFIGS[name][0]
        w = tiny.load_weights(model_folders[name])
        for k_ in w:
            if k_.endswith("o_proj.weight") or k_.endswith("down_proj.weight") or k_.endswith("o_proj.bias"):
                w[k_] = torch.zeros_like(w[k_])
        toks = tiny.prompt(name, 6)
        head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
        want = P.linear(P.rmsnorm(w["model.embed_tokens.weight"][toks], w["model.norm.weight"], cfg["rms_norm_eps"]), head)
        assert torch.allclose(P.forward(cfg, w, toks), want, atol=1e-12)
    # tying: config A has no lm_head.weight and uses the embedding
    assert "lm_head.weight" not in tiny.load_weights(model_folders["A"])


def test_qk_norm_gains_matter_and_v_is_not_normalised(model_folders):
    cfg = tiny.CONFIGS["B"][0]
    w = tiny.load_weights(model_folders["B"])
    toks = tiny.prompt("B", 12)
    base = P.forward(cfg, w, toks)
    w2 = dict(w)
    w2["model.layers.1.self_attn.q_norm.weight"] = w["model.layers.1.self_attn.q_norm.weight"] * 1.5
    assert (P.forward(cfg, w2, toks) - base).abs().max() > 1e-6, "the q gain matters"
    # scaling q_proj rows by a constant changes nothing: the per-head norm (eps aside) removes it
    w3 = dict(w)
    w3["model.layers.1.self_attn.q_proj.weight"] = w["model.layers.1.self_attn.q_proj.weight"] * 64.0
    assert (P.forward(cfg, w3, toks) - base).abs().max() < 1e-3 * base.abs().max()
    # v is not normalised: scaling v_proj does change the result
    w4 = dict(w)
    w4["model.layers.1.self_attn.v_proj.weight"] = w["model.layers.1.self_attn.v_proj.weight"] * 2.0
    assert (P.forward(cfg, w4, toks) - base).abs().max() > 1e-4
    # rows do not see the future; a prefix gives the same logits
    assert torch.allclose(P.forward(cfg, w, toks[:7]), base[:7], atol=1e-12)


def _attention_block_with(order, xb, w, prefix, cfg, positions):
    """The attention block put together from the plain parts with the q/k preparation in a given order: ``norm, rotate``
    is what ``P.attention_block`` does; the others are the plausible mistakes the invariants below must reject."""
    p = prefix + ".self_attn."
    T, H, Hkv, hd = xb.shape[0], cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    cos, sin = P.rope_angles(positions, cfg["rotary_dim"], cfg["theta"], cfg["rope_scaling"], cfg["max_pos"])

    def prep(name, heads, gain):
        y = P.linear(xb, w[p + name + "_proj.weight"], None if order == "norm, bias, rotate" or not cfg["bias"]
                     else w[p + name + "_proj.bias"]).view(T, heads, hd)
        if order == "rotate, norm":
            return P.rmsnorm(P.apply_rope(y, cos, sin), gain, cfg["eps"])
        y = P.rmsnorm(y, gain, cfg["eps"])
        if order == "norm, bias, rotate" and cfg["bias"]:
            y = y + w[p + name + "_proj.bias"].view(heads, hd)
        return P.apply_rope(y, cos, sin)
    q = prep("q", H, w[p + "q_norm.weight"])
    k = prep("k", Hkv, w[p + "k_norm.weight"])
    v = P.linear(xb, w[p + "v_proj.weight"], w[p + "v_proj.bias"] if cfg["bias"] else None).view(T, Hkv, hd)
    scale = float(torch.tensor(1.0 / math.sqrt(hd), dtype=torch.float32))
    att = P.attention(q, k, v, scale, 0, int(positions[0])).reshape(T, H * hd)
    return P.linear(att, w[p + "o_proj.weight"], w.get(p + "o_proj.bias") if cfg["bias"] else None)


def test_shifting_all_positions_changes_nothing_only_if_the_rotation_comes_last(model_folders):
    """Scores depend on the distance between query and key only (docs/05-transformer-math.md:509-524: key at 2, query
    at 5, unchanged when both shift by 10). A rotation is orthogonal, so that holds whatever comes before it; a gain
    applied AFTER the rotation weighs the two halves of a rotated pair differently and breaks it. With q and k gains
    that differ within every pair, the block's output at positions p.. and p+10.. is equal only for norm -> rotate."""
    cfg = P.read_config(tiny.CONFIGS["B"][0])
    w = dict(tiny.load_weights(model_folders["B"]))
    gen = torch.Generator().manual_seed(3)
    for n in ("q_norm", "k_norm"):
        w[f"model.layers.1.self_attn.{n}.weight"] = torch.rand(cfg["head_dim"], generator=gen, dtype=D) * 2.5 + 0.25
    xb = torch.randn(11, cfg["dim"], generator=gen, dtype=D)
    here, there = torch.arange(11), torch.arange(11) + 10
    a = P.attention_block(xb, w, "model.layers.1", cfg, 1, here)
    b = P.attention_block(xb, w, "model.layers.1", cfg, 1, there)
    assert (a - b).abs().max() < 1e-6 * a.abs().max()  # the table is rounded to float32: not to the last bit
    # the helper agrees with the plain block in the right order, and the wrong order is told apart by a wide margin
    assert torch.allclose(_attention_block_with("norm, rotate", xb, w, "model.layers.1", cfg, here), a, atol=1e-12)
    wrong_a = _attention_block_with("rotate, norm", xb, w, "model.layers.1", cfg, here)
    wrong_b = _attention_block_with("rotate, norm", xb, w, "model.layers.1", cfg, there)
    assert (wrong_a - wrong_b).abs().max() > 1e-2 * a.abs().max()
    # a scale of theta away from the config's does not pass either: the angles are the table's, per position
    assert (P.attention_block(xb, w, "model.layers.1", cfg, 1, there * 2) - a).abs().max() > 1e-3 * a.abs().max()


def test_the_bias_is_inside_the_head_norm():
    """q = norm(W x + b): multiplying W_q AND b_q by 64 leaves the normalised q, and so the logits, unchanged (eps -> 0);
    multiplying the bias alone changes them. With the bias added after the norm the first would change the logits
    (cpu/CpuBackend.java:430-436: bias right after the projection; :595-608: the norm after that)."""
    cfg_d = dict(tiny.TINY_C, rms_norm_eps=1e-12)
    from jllm_serve_amd.weights.random_init import random_source
    src = random_source(cfg_d, seed=11)
    w = {n: src.get(n).to(D) for n in src.names()}
    toks = tiny.prompt("C", 14, seed=2)
    base = P.forward(cfg_d, w, toks)
    both, bias_only = dict(w), dict(w)
    for n in ("q", "k"):
        for l in range(cfg_d["num_hidden_layers"]):
            key = f"model.layers.{l}.self_attn.{n}_proj."
            both[key + "weight"], both[key + "bias"] = w[key + "weight"] * 64, w[key + "bias"] * 64
            bias_only[key + "bias"] = w[key + "bias"] * 64
    scale = base.abs().max()
    assert (P.forward(cfg_d, both, toks) - base).abs().max() < 1e-9 * scale
    assert (P.forward(cfg_d, bias_only, toks) - base).abs().max() > 1e-3 * scale
    # the mistake this rejects: norm first, bias afterwards
    cfg = P.read_config(cfg_d)
    xb = torch.randn(9, cfg["dim"], dtype=D, generator=torch.Generator().manual_seed(1))
    pos = torch.arange(9)
    right = P.attention_block(xb, w, "model.layers.0", cfg, 0, pos)
    assert (P.attention_block(xb, both, "model.layers.0", cfg, 0, pos) - right).abs().max() < 1e-9 * right.abs().max()
    wrong = _attention_block_with("norm, bias, rotate", xb, w, "model.layers.0", cfg, pos)
    wrong64 = _attention_block_with("norm, bias, rotate", xb, both, "model.layers.0", cfg, pos)
    assert (wrong64 - wrong).abs().max() > 1e-2 * right.abs().max()


def test_order_of_bias_norm_and_rotation_in_a_case_computed_by_hand():
    """One head of two dims, so that everything can be written out: q = rope(norm(W x + b)) in exactly this order
    (cpu/CpuBackend.java:430-436 bias right after the projection, :608-614 the per-head norm with the model's eps
    before the rotation; docs/05-transformer-math.md:428-434). The gains of the two dims differ, so norm-then-rotate
    and rotate-then-norm give different numbers, and so do bias-then-norm and norm-then-bias, and another eps.
    The reference holds no vector for these orders: they are pinned by its text, and this test pins the plain
    implementation to that text."""
    eps = 0.25
    cfg = P.read_config(dict(num_attention_heads=1, num_key_value_heads=1, hidden_size=2, head_dim=2, num_hidden_layers=1,
                             vocab_size=4, intermediate_size=2, rms_norm_eps=eps, rope_theta=1.0, attention_bias=True))
    eye = torch.eye(2, dtype=D)
    gq, gk = t([2.0, 0.5]), t([0.5, 1.5])
    bq, bk, bv = t([-0.9, 0.9]), t([0.2, -0.3]), t([0.0, 0.0])
    w = {"L.self_attn.q_proj.weight": eye, "L.self_attn.k_proj.weight": eye, "L.self_attn.v_proj.weight": eye,
         "L.self_attn.o_proj.weight": eye, "L.self_attn.q_proj.bias": bq, "L.self_attn.k_proj.bias": bk,
         "L.self_attn.v_proj.bias": bv, "L.self_attn.o_proj.bias": t([0.0, 0.0]), "L.self_attn.q_norm.weight": gq,
         "L.self_attn.k_norm.weight": gk}
    x = t([[0.5, 1.9], [0.6, -1.0]])  # positions 0 and 1 (values found by a search for a case that separates the orders well)
    got = P.attention_block(x, w, "L", cfg, 0, torch.arange(2))

    def by_hand(order, bias_first=True, e=eps):
        def prep(v, b, g, p):  # one 2-vector
            v = [v[0] + b[0], v[1] + b[1]] if bias_first else list(v)
            c, s_ = math.cos(p * 1.0), math.sin(p * 1.0)  # theta = 1: the one pair turns by p radians

            def norm(u):
                r = 1.0 / math.sqrt((u[0] * u[0] + u[1] * u[1]) / 2 + e)
                return [u[0] * r * g[0], u[1] * r * g[1]]

            def rot(u):
                return [u[0] * c - u[1] * s_, u[1] * c + u[0] * s_]
            v = rot(norm(v)) if order == "norm, rotate" else norm(rot(v))
            return v if bias_first else [v[0] + b[0], v[1] + b[1]]
        xs = x.tolist()
        q1 = prep(xs[1], bq.tolist(), gq.tolist(), 1)
        k0, k1 = prep(xs[0], bk.tolist(), gk.tolist(), 0), prep(xs[1], bk.tolist(), gk.tolist(), 1)
        scale = 1.0 / math.sqrt(2)
        s0, s1 = (q1[0] * k0[0] + q1[1] * k0[1]) * scale, (q1[0] * k1[0] + q1[1] * k1[1]) * scale
        m = max(s0, s1)
        e0, e1 = math.exp(s0 - m), math.exp(s1 - m)
        p0, p1 = e0 / (e0 + e1), e1 / (e0 + e1)
        return [p0 * xs[0][0] + p1 * xs[1][0], p0 * xs[0][1] + p1 * xs[1][1]]  # v = x (identity, zero bias)

    right = by_hand("norm, rotate")
    assert torch.allclose(got[1], t(right), atol=1e-6)
    assert torch.allclose(got[0], x[0])  # position 0 sees only itself
    for wrong in (by_hand("rotate, norm"), by_hand("norm, rotate", bias_first=False), by_hand("norm, rotate", e=1e-6)):
        assert max(abs(a - b) for a, b in zip(right, wrong)) > 0.3, "the case must tell the orders apart"


def test_greedy_takes_the_lowest_index_on_ties():
    """plain.greedy through a model whose logits tie: token 1 and token 2 have the same head row, and the lower index
    must be generated (sampling/Sampler.java:458-466)."""
    cfg = dict(tiny.TINY_A)
    torch.manual_seed(0)
    from jllm_serve_amd.weights.random_init import random_source
    src = random_source(cfg, seed=5)
    w = {n: src.get(n).to(D) for n in src.names()}
    emb = w["model.embed_tokens.weight"]  # tied: the head is the embedding
    z = P.forward(cfg, w, [3, 9, 27])[-1]
    best = int(torch.argmax(z))
    other = (best + 5) % emb.shape[0]
    lo, hi = min(best, other), max(best, other)
    emb[lo] = emb[best].clone()
    emb[hi] = emb[lo].clone()
    z2 = P.forward(cfg, w, [3, 9, 27])[-1]
    if best not in (3, 9, 27) and other not in (3, 9, 27):  # the prompt's own rows were not touched
        assert z2[lo] == z2[hi] == z2.max()
    assert P.greedy(cfg, w, [3, 9, 27], 1) == [int((z2 == z2.max()).nonzero()[0])]
    assert int((z2 == z2.max()).nonzero()[0]) == lo or z2[lo] < z2.max()
