"""Safetensors by name, the one error for everything wrong, the storage rule,
and random weights (no GPU)."""
import json
import os
import struct

import pytest
import torch

from torchless_rs_amd.config import config_from_dict
from torchless_rs_amd.models import model_spec_for
from torchless_rs_amd.weights import (ModelFiles, SafetensorsError, SafetensorsFile, TensorDict,
                                      WeightBindingError, WeightSpec, bind_weights, random_tensors,
                                      stored_to_resident, write_random_model, write_safetensors)
from util import TINY_A, TINY_B, read_model_dir


def test_round_trip(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(4).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int64).view(2, 3), "d": torch.randn(2, 2).to(torch.float16)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, t, {"k": "v"})
    f = SafetensorsFile(p)
    assert sorted(f.names()) == ["a", "b", "c", "d"] and f.metadata == {"k": "v"}
    for k, v in t.items():
        assert f.dtype(k) == v.dtype and f.shape(k) == tuple(v.shape)
        assert torch.equal(f.tensor(k), v)
    # the layout is the published one: u64 length, JSON, data
    raw = open(p, "rb").read()
    (n,) = struct.unpack("<Q", raw[:8])
    hdr = json.loads(raw[8:8 + n])
    assert hdr["a"]["dtype"] == "F32" and hdr["b"]["dtype"] == "BF16" and hdr["a"]["shape"] == [3, 5]
    b, e = hdr["a"]["data_offsets"]
    assert torch.equal(torch.frombuffer(bytearray(raw[8 + n + b:8 + n + e]), dtype=torch.float32).view(3, 5), t["a"])


def _write_raw(path, header: dict, data: bytes = b""):
    hj = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + data)


def test_malformed_files(tmp_path):
    p = str(tmp_path / "f.safetensors")
    with pytest.raises(SafetensorsError, match="cannot open"):
        SafetensorsFile(p)
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="8-byte"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="past the end"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 2) + b"[]")
    with pytest.raises(SafetensorsError, match="object"):
        SafetensorsFile(p)
    _write_raw(p, {"t": {"dtype": "Q9", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        SafetensorsFile(p)
    _write_raw(p, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="outside the file"):
        SafetensorsFile(p)
    _write_raw(p, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="need"):
        SafetensorsFile(p)
    # a negative shape whose product would pass the count of bytes; offsets that are no integers
    _write_raw(p, {"t": {"dtype": "U8", "shape": [-2, -3], "data_offsets": [0, 6]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="negative dimension"):
        SafetensorsFile(p)
    _write_raw(p, {"t": {"dtype": "U8", "shape": [4], "data_offsets": [0.0, 4.0]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="must be integers"):
        SafetensorsFile(p)
    _write_raw(p, {"t": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]},
                   "u": {"dtype": "U8", "shape": [4], "data_offsets": [2, 6]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="overlaps"):
        SafetensorsFile(p)
    with pytest.raises(SafetensorsError, match="neither"):
        ModelFiles(str(tmp_path / "nothing"))


def test_an_index_cannot_name_files_outside_the_folder(tmp_path):
    inside, outside = tmp_path / "model", tmp_path / "elsewhere"
    inside.mkdir()
    outside.mkdir()
    write_safetensors(str(outside / "x.safetensors"), {"a": torch.ones(2)})
    for shard in ("../elsewhere/x.safetensors", str(outside / "x.safetensors"), "sub/x.safetensors", ".."):
        (inside / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": shard}}))
        with pytest.raises(SafetensorsError, match="plain file name"):
            ModelFiles(str(inside))
    os.symlink(str(outside / "x.safetensors"), str(inside / "link.safetensors"))
    (inside / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "link.safetensors"}}))
    with pytest.raises(SafetensorsError, match="outside"):
        ModelFiles(str(inside))
    (inside / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": 3}}))
    with pytest.raises(SafetensorsError, match="file names"):
        ModelFiles(str(inside))


def test_sharded_folder(tmp_path):
    write_safetensors(str(tmp_path / "m-1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "m-2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "m-1.safetensors", "b": "m-2.safetensors"}}))
    m = ModelFiles(str(tmp_path))
    assert sorted(m.names()) == ["a", "b"] and torch.equal(m.tensor("b"), torch.zeros(3))


def test_one_error_lists_everything():
    spec = model_spec_for(config_from_dict(TINY_A)).weight_specs()
    t = random_tensors(spec, 0, dtype=torch.float32)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["lm_head.weight"]
    t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63)
    t["model.norm.weight"] = torch.zeros(65)
    t["model.layers.7.extra.weight"] = torch.zeros(1)
    t["model.embed_tokens.weight"] = torch.zeros(256, 64, dtype=torch.int32)
    with pytest.raises(WeightBindingError) as ei:
        bind_weights(spec, TensorDict(t), torch.float32, None)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "lm_head.weight"]
    assert e.unexpected == ["model.layers.7.extra.weight"]
    assert sorted(n for n, _, _ in e.mismatched) == ["model.layers.0.self_attn.q_proj.weight", "model.norm.weight"]
    assert ("model.layers.0.self_attn.q_proj.weight", (64, 63), (64, 64)) in e.mismatched
    assert [n for n, _ in e.bad_dtype] == ["model.embed_tokens.weight"]
    msg = str(e)
    for word in ("missing", "unexpected", "wrong shapes", "lm_head.weight", "extra.weight", "[64, 63]"):
        assert word in msg


def test_ignored_names_and_full_bind():
    spec = model_spec_for(config_from_dict(TINY_B))
    t = random_tensors(spec.weight_specs(), 2, 0.05, 0.1)
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    out = bind_weights(spec.weight_specs(), TensorDict(t), torch.bfloat16, None, spec.ignore_tensors)
    assert list(out) == list(spec.weight_specs())


def test_storage_rule():
    bf, f16, f32, i64 = (torch.ones(2, dtype=d) for d in (torch.bfloat16, torch.float16, torch.float32, torch.int64))
    assert stored_to_resident(bf, torch.bfloat16).dtype == torch.bfloat16
    assert stored_to_resident(f16, torch.bfloat16).dtype == torch.bfloat16
    assert stored_to_resident(f32, torch.bfloat16).dtype == torch.float32      # stored in 32 bits: stays
    assert stored_to_resident(i64, torch.bfloat16).dtype == torch.int32
    assert stored_to_resident(bf, torch.float32).dtype == torch.float32
    assert stored_to_resident(i64, torch.float32).dtype == torch.int32


def test_random_model_folder(tmp_path):
    d1 = write_random_model(str(tmp_path / "m1"), dict(TINY_B), seed=2, std=0.05, norm_std=0.1)
    d2 = write_random_model(str(tmp_path / "m2"), dict(TINY_B), seed=2, std=0.05, norm_std=0.1)
    d3 = write_random_model(str(tmp_path / "m3"), dict(TINY_B), seed=3, std=0.05, norm_std=0.1)
    assert sorted(os.listdir(d1)) == ["config.json", "model.safetensors"]
    c1, t1 = read_model_dir(d1)
    _, t2 = read_model_dir(d2)
    _, t3 = read_model_dir(d3)
    assert c1["head_dim"] == 32 and c1["architectures"] == ["MistralForCausalLM"]
    assert all(torch.equal(t1[k], t2[k]) for k in t1)                          # the seed decides
    assert not torch.equal(t1["lm_head.weight"], t3["lm_head.weight"])
    w = t1["model.layers.1.mlp.down_proj.weight"].float()
    assert w.dtype == torch.float32 and abs(float(w.std()) - 0.05) < 0.005 and abs(float(w.mean())) < 0.005
    n = t1["model.layers.0.input_layernorm.weight"].float()
    assert abs(float(n.mean()) - 1) < 0.05 and 0.05 < float(n.std()) < 0.2
    dA = write_random_model(str(tmp_path / "a"), dict(TINY_A), seed=0, dtype=torch.float32)
    _, tA = read_model_dir(dA)
    assert tA["model.norm.weight"].dtype == torch.float32 and bool((tA["model.norm.weight"] == 1).all())
    # and the folder loads back through the framework's own reader and binder
    spec = model_spec_for(config_from_dict(c1))
    out = bind_weights(spec.weight_specs(), ModelFiles(d1), torch.bfloat16, None, spec.ignore_tensors)
    assert out["lm_head.weight"].dtype == torch.bfloat16 and torch.equal(out["lm_head.weight"], t1["lm_head.weight"])
