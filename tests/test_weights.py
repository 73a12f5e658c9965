import json
import os
import struct

import pytest
import torch

from kipp_amd.config import parse_config
from kipp_amd.engine.model import model_params
from kipp_amd.runtime import device_dtype
from kipp_amd.weights import (SafetensorsError, WeightError, check_tensors, random_tensors, read_file,
                              read_model_tensors, write_file, write_random_model)


def test_own_reader_and_writer_agree_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    tensors = {"a.weight": torch.randn(5, 7).bfloat16(), "b": torch.randn(3), "idx": torch.arange(6, dtype=torch.int32).reshape(2, 3),
               "s": torch.tensor(2.5)}
    write_file(str(tmp_path / "ours.safetensors"), tensors, metadata={"format": "pt"})
    theirs = load_file(str(tmp_path / "ours.safetensors"))
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    ours = read_file(str(tmp_path / "theirs.safetensors"))
    for name, t in tensors.items():
        assert torch.equal(theirs[name], t) and torch.equal(ours[name], t) and ours[name].dtype == t.dtype


def test_random_model_is_deterministic_and_order_independent(tmp_path, tiny_configs):
    a = write_random_model(str(tmp_path / "a"), tiny_configs["a"], seed=5)
    b = write_random_model(str(tmp_path / "b"), tiny_configs["a"], seed=5)
    c = write_random_model(str(tmp_path / "c"), tiny_configs["a"], seed=6)
    ta, tb, tc = (read_model_tensors(d) for d in (a, b, c))
    expected = model_params(parse_config(tiny_configs["a"])[1].model_spec())
    assert set(ta) == set(expected) and "lm_head.weight" not in ta
    assert all(torch.equal(ta[n], tb[n]) for n in ta) and not torch.equal(ta["model.norm.weight"], tc["model.norm.weight"])
    one = random_tensors({"model.norm.weight": expected["model.norm.weight"]}, 5)["model.norm.weight"]
    assert torch.equal(one, ta["model.norm.weight"])           # a tensor's values depend on (seed, name) only
    assert ta["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert abs(float(ta["model.embed_tokens.weight"].float().std()) - 0.02) < 0.002
    assert abs(float(ta["model.norm.weight"].float().mean()) - 1.0) < 0.05
    cfg = json.load(open(os.path.join(a, "config.json")))
    assert cfg["architectures"] == ["Qwen3ForCausalLM"] and cfg["torch_dtype"] == "bfloat16"
    untied = read_model_tensors(write_random_model(str(tmp_path / "u"), tiny_configs["b"], seed=1, dtype="float32"))
    assert untied["lm_head.weight"].shape == (509, 80) and untied["lm_head.weight"].dtype == torch.float32


def test_one_error_lists_missing_unexpected_and_wrong(tmp_path, tiny_configs):
    folder = write_random_model(str(tmp_path / "m"), tiny_configs["a"], seed=5)
    tensors = dict(read_model_tensors(folder))
    expected = model_params(parse_config(tiny_configs["a"])[1].model_spec())
    check_tensors(folder, tensors, expected)
    del tensors["model.layers.1.mlp.up_proj.weight"], tensors["model.norm.weight"]
    tensors["lm_head.weight"] = torch.zeros(256, 64)          # tied model: a head of its own is unexpected
    tensors["model.layers.0.extra.bias"] = torch.zeros(3)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64)
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16, dtype=torch.int32)
    with pytest.raises(WeightError) as e:
        check_tensors(folder, tensors, expected)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["lm_head.weight", "model.layers.0.extra.bias"]
    assert len(err.wrong) == 2
    text = str(err)
    for needle in ("missing tensors (2)", "unexpected tensors (2)", "wrong shape or type (2)", "k_proj.weight: shape (64, 64), expected (32, 64)",
                   "q_norm.weight: type torch.int32"):
        assert needle in text


def test_malformed_files_are_refused(tmp_path):
    path = str(tmp_path / "model.safetensors")
    write_file(path, {"w": torch.zeros(4, 4)})
    raw = open(path, "rb").read()
    open(path, "wb").write(raw[:-8])
    with pytest.raises(SafetensorsError, match="outside the file"):
        read_file(path)
    open(path, "wb").write(raw[:5])
    with pytest.raises(SafetensorsError, match="truncated"):
        read_file(path)
    open(path, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="does not fit"):
        read_file(path)
    header = json.dumps({"w": {"dtype": "F32", "shape": [4, 4], "data_offsets": [0, 60]}}).encode()
    open(path, "wb").write(struct.pack("<Q", len(header)) + header + b"\0" * 64)
    with pytest.raises(SafetensorsError, match="needs 64"):
        read_file(path)
    header = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]},
                         "b": {"dtype": "F32", "shape": [4], "data_offsets": [8, 24]}}).encode()
    open(path, "wb").write(struct.pack("<Q", len(header)) + header + b"\0" * 24)
    with pytest.raises(SafetensorsError, match="overlap"):
        read_file(path)
    with pytest.raises(SafetensorsError, match="neither"):
        read_model_tensors(str(tmp_path / "nothing"))


def test_sharded_folder(tmp_path):
    write_file(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_file(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    t = read_model_tensors(str(tmp_path))
    assert set(t) == {"a", "b"} and t["b"].shape == (3,)


def test_device_types():
    bf, f32, f16, i64 = torch.bfloat16, torch.float32, torch.float16, torch.int64
    assert device_dtype(bf, "float", "bfloat16") == bf            # kept in bfloat16
    assert device_dtype(f32, "float", "bfloat16") == f32          # a tensor stored in 32-bit stays so
    assert device_dtype(f16, "float", "bfloat16") == f32
    assert device_dtype(bf, "float", "float32") == f32
    assert device_dtype(i64, "int", "bfloat16") == torch.int32    # integer tables as int32
