"""The safetensors reader's header checks, loading by name, the one error for bad checkpoints, random weights."""
import json
import os
import struct

import pytest
import torch

import tiny
from jllm_serve_amd.weights import (SafetensorsError, SafetensorsFile, SafetensorsSource, WeightError, check,
                                    storage_dtype, write_random_model, write_safetensors)
from jllm_serve_amd.weights.random_init import model_weight_specs, random_source


def raw_file(path, header, data=b"", pad=True):
    blob = header if isinstance(header, bytes) else json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        f.write(data)


def test_roundtrip_and_views(tmp_path):
    p = str(tmp_path / "t.safetensors")
    a = torch.arange(12, dtype=torch.float32).view(3, 4)
    b = torch.randn(5, 2).to(torch.bfloat16)
    c = torch.tensor([1, -2, 3], dtype=torch.int64)
    write_safetensors(p, {"a": a, "b": b, "c": c}, metadata={"k": "v"})
    f = SafetensorsFile(p)
    assert set(f.names()) == {"a", "b", "c"} and f.metadata == {"k": "v"}
    assert torch.equal(f.tensor("a"), a) and torch.equal(f.tensor("b"), b) and torch.equal(f.tensor("c"), c)
    from safetensors import safe_open  # the format package reads what we wrote
    with safe_open(p, framework="pt") as g:
        assert torch.equal(g.get_tensor("b"), b)
    with pytest.raises(SafetensorsError, match="tensor not found: zz"):
        f.tensor("zz")


@pytest.mark.parametrize("header,data,msg", [
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 8, "do not fit"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4, "do not fit"),
    ({"a": {"dtype": "F32", "shape": [-2], "data_offsets": [0, 8]}}, b"\0" * 8, "negative dimension"),
    ({"a": {"dtype": "Q9", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, "unsupported dtype"),
    ({"a": {"shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, "no dtype"),
    ({"a": {"dtype": "F32", "shape": [2]}}, b"\0" * 8, "malformed entry"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]},
      "b": {"dtype": "F32", "shape": [1], "data_offsets": [2, 6]}}, b"\0" * 8, "overlap"),
    (b'{"a": ', b"", "invalid header JSON"),
    (b'{"a": {"dtype":"F32","shape":[1],"data_offsets":[0,4]}, "a": {"dtype":"F32","shape":[1],"data_offsets":[4,8]}}',
     b"\0" * 8, "duplicate tensor"),
])
def test_header_errors(tmp_path, header, data, msg):
    p = str(tmp_path / "bad.safetensors")
    raw_file(p, header, data)
    with pytest.raises(SafetensorsError, match=msg):
        SafetensorsFile(p)


def test_file_level_errors(tmp_path):
    p = str(tmp_path / "small.safetensors")
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="too small"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(SafetensorsError, match="no .safetensors files"):
        SafetensorsSource(str(empty))


def test_sharded_folder(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), {"x": torch.ones(2)})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"y": torch.zeros(3)})
    src = SafetensorsSource(str(tmp_path))
    assert sorted(src.names()) == ["x", "y"] and src.shape("y") == (3,)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "s1.safetensors"}}))
    assert SafetensorsSource(str(tmp_path)).names() == ["x"]
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "../s1.safetensors"}}))
    with pytest.raises(SafetensorsError, match="bad shard name"):
        SafetensorsSource(str(tmp_path))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"nothing": 1}))
    with pytest.raises(SafetensorsError, match="weight_map"):
        SafetensorsSource(str(tmp_path))
    os.remove(tmp_path / "model.safetensors.index.json")
    write_safetensors(str(tmp_path / "s3.safetensors"), {"x": torch.ones(2)})
    with pytest.raises(SafetensorsError, match="duplicate tensor 'x'"):
        SafetensorsSource(str(tmp_path))


def test_random_model_folder_loads_and_is_seeded(tmp_path):
    d1 = write_random_model(str(tmp_path / "m1"), tiny.TINY_A, seed=0)
    d2 = write_random_model(str(tmp_path / "m2"), tiny.TINY_A, seed=0)
    d3 = write_random_model(str(tmp_path / "m3"), tiny.TINY_A, seed=1)
    s1, s2, s3 = SafetensorsSource(d1), SafetensorsSource(d2), SafetensorsSource(d3)
    cfg, specs = model_weight_specs(tiny.TINY_A)
    check(specs, s1)
    assert "lm_head.weight" not in s1.names(), "tied embeddings: no output head in the file"
    assert len(s1.names()) == 1 + 2 * 11 + 1  # embed, 11 tensors a layer (4 proj, 2 qk norms, 2 norms, 3 mlp), final norm
    for n in s1.names():
        assert torch.equal(s1.get(n), s2.get(n)) and s1.dtype(n) == torch.bfloat16
    assert not torch.equal(s1.get("model.embed_tokens.weight"), s3.get("model.embed_tokens.weight"))
    e = s1.get("model.embed_tokens.weight").float()
    assert abs(e.std().item() - 0.02) < 0.002 and abs(e.mean().item()) < 0.002
    g = s1.get("model.layers.0.self_attn.q_norm.weight").float()
    assert abs(g.mean().item() - 1.0) < 0.1 and g.std().item() > 0.01, "gains are 1 + N(0, 0.1), not exactly 1"
    assert json.load(open(os.path.join(d1, "config.json"))) == tiny.TINY_A
    b = SafetensorsSource(write_random_model(str(tmp_path / "m4"), tiny.TINY_C, seed=2))
    assert "model.layers.3.self_attn.o_proj.bias" in b.names() and "lm_head.weight" in b.names()
    unit = random_source(tiny.TINY_A, 0, gain_std=0.0).get("model.norm.weight")
    assert torch.equal(unit.float(), torch.ones(64))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(str(tmp_path / "m"), tiny.TINY_B, seed=1)
    src = SafetensorsSource(d)
    tensors = {n: src.get(n).clone() for n in src.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 95, dtype=torch.bfloat16)
    tensors["model.layers.2.self_attn.q_norm.weight"] = torch.zeros(16, dtype=torch.bfloat16)
    tensors["model.layers.7.mlp.up_proj.weight"] = torch.zeros(1, dtype=torch.bfloat16)
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    write_safetensors(os.path.join(bad, "model.safetensors"), tensors)
    _, specs = model_weight_specs(tiny.TINY_B)
    with pytest.raises(WeightError) as ei:
        check(specs, SafetensorsSource(bad), where="test")
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["model.layers.0.self_attn.k_proj.weight",
                                                      "model.layers.2.self_attn.q_norm.weight"]
    text = str(e)
    for s in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "[64, 95], expected [64, 96]"):
        assert s in text
    # an untied model without lm_head.weight: missing; a tied one with it: accepted (ModelWeights.java:36-43)
    t2 = {n: src.get(n) for n in src.names() if n != "lm_head.weight"}
    write_safetensors(os.path.join(bad, "model.safetensors"), t2)
    with pytest.raises(WeightError, match="lm_head.weight"):
        check(specs, SafetensorsSource(bad))


def test_storage_rule():
    assert storage_dtype(torch.bfloat16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype(torch.float16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype(torch.float32, torch.bfloat16) == torch.float32, "a tensor stored in 32-bit stays so"
    assert storage_dtype(torch.bfloat16, torch.float32) == torch.float32
    assert storage_dtype(torch.int64, torch.bfloat16) == torch.int32
