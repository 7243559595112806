"""Safetensors reading and the loader's error reporting (no GPU)."""

import json
import os
import struct

import numpy as np
import pytest
import torch

from flyweight_amd.config import config_from_dict
from flyweight_amd.engine.model import declared_tensors
from flyweight_amd.weights import (SafetensorsError, SafetensorsFile, TensorDecl, WeightError, load_tensors,
                                   read_header, storage_dtype, write_file, write_random_model)
from helpers import TINY_A, TINY_B, make_model

CPU = torch.device("cpu")


def _raw(path, header: dict, payload: bytes, header_len=None):
    raw = json.dumps(header).encode()
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw) if header_len is None else header_len))
        handle.write(raw)
        handle.write(payload)


def test_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32)}
    path = str(tmp_path / "x.safetensors")
    write_file(path, tensors)
    with SafetensorsFile(path) as handle:
        for name, value in tensors.items():
            assert torch.equal(handle.tensor(name), value)
    from safetensors.torch import load_file
    for name, value in load_file(path).items():
        assert torch.equal(value, tensors[name])


def test_header_checks(tmp_path):
    path = str(tmp_path / "bad.safetensors")
    _raw(path, {}, b"", header_len=1 << 40)
    with pytest.raises(SafetensorsError, match="truncated"):
        read_header(path)
    _raw(path, {"t": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}, b"\0\0")
    with pytest.raises(SafetensorsError, match="F8_E4M3"):
        read_header(path)
    _raw(path, {"t": {"dtype": "F32", "shape": [2], "data_offsets": [8, 0]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="inverted"):
        read_header(path)
    _raw(path, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="truncated"):
        read_header(path)
    _raw(path, {"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 12"):
        read_header(path)
    _raw(path, {"__metadata__": {"k": "v"}, "t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8)
    assert list(read_header(path)) == ["t"]
    with open(path, "wb") as handle:
        handle.write(b"\1\2\3")
    with pytest.raises(SafetensorsError, match="too short"):
        read_header(path)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_model(str(tmp_path / "m"), "A")
    declared = declared_tensors(config_from_dict(TINY_A).model_spec())
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as handle:
        tensors = {name: handle.tensor(name) for name in handle.names()}
    del tensors["model.layers.1.self_attn.q_layernorm.weight"]
    del tensors["model.layers.0.conv.conv.weight"]
    tensors["model.layers.9.extra.weight"] = torch.zeros(2)
    tensors["lm_head.weight"] = torch.zeros(256, 64)              # tied model: the head is not expected
    tensors["model.layers.2.feed_forward.w2.weight"] = torch.zeros(64, 161)
    write_file(path, tensors)
    with pytest.raises(WeightError) as error:
        load_tensors(folder, declared, torch.float32, CPU)
    e = error.value
    assert e.missing == ["model.layers.0.conv.conv.weight", "model.layers.1.self_attn.q_layernorm.weight"]
    assert e.unexpected == ["lm_head.weight", "model.layers.9.extra.weight"]
    assert e.wrong_shape == [("model.layers.2.feed_forward.w2.weight", (64, 160), (64, 161))]
    text = str(e)
    for piece in ("missing tensors (2)", "unexpected tensors (2)", "wrong shapes (1)", "expected [64, 160] found [64, 161]"):
        assert piece in text


def test_untied_model_requires_its_head(tmp_path):
    folder = make_model(str(tmp_path / "m"), "B")
    declared = declared_tensors(config_from_dict(TINY_B).model_spec())
    assert "lm_head.weight" in declared
    assert declared["model.layers.1.conv.in_proj.bias"].shape == (288,)
    assert declared["model.layers.1.conv.conv.weight"].shape == (96, 1, 4)
    tensors = load_tensors(folder, declared, torch.bfloat16, CPU)
    assert set(tensors) == set(declared)


def test_storage_rule(tmp_path):
    # bfloat16 stays bfloat16, 32-bit stays 32-bit, vectors are widened, a float32 run widens all
    assert storage_dtype("matrix", torch.bfloat16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype("matrix", torch.float32, torch.bfloat16) == torch.float32
    assert storage_dtype("matrix", torch.float16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype("matrix", torch.bfloat16, torch.float32) == torch.float32
    assert storage_dtype("vector", torch.bfloat16, torch.bfloat16) == torch.float32
    assert storage_dtype("table", torch.int64, torch.bfloat16) == torch.int32
    folder = make_model(str(tmp_path / "m"), "A")
    declared = declared_tensors(config_from_dict(TINY_A).model_spec())
    loaded = load_tensors(folder, declared, torch.bfloat16, CPU)
    assert loaded["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert loaded["model.layers.0.operator_norm.weight"].dtype == torch.float32
    assert loaded["model.layers.0.conv.conv.weight"].dtype == torch.float32
    as32 = load_tensors(folder, declared, torch.float32, CPU)
    assert all(t.dtype == torch.float32 for t in as32.values())
    assert torch.equal(as32["model.embed_tokens.weight"], loaded["model.embed_tokens.weight"].float())
    declared_table = {"ids": TensorDecl((4,), role="table")}
    os.makedirs(tmp_path / "t")
    write_file(str(tmp_path / "t" / "model.safetensors"), {"ids": torch.arange(4, dtype=torch.int64)})
    assert load_tensors(str(tmp_path / "t"), declared_table, torch.bfloat16, CPU)["ids"].dtype == torch.int32


def test_random_weights_are_seeded_and_complete(tmp_path):
    config = config_from_dict(TINY_B)
    one = write_random_model(str(tmp_path / "one"), config, 5)
    two = write_random_model(str(tmp_path / "two"), config, 5)
    three = write_random_model(str(tmp_path / "three"), config, 6)
    assert sorted(os.listdir(one)) == ["config.json", "model.safetensors"]
    a, b, c = (read_header(os.path.join(f, "model.safetensors")) for f in (one, two, three))
    assert set(a) == set(declared_tensors(config.model_spec()))
    with SafetensorsFile(os.path.join(one, "model.safetensors")) as x, \
            SafetensorsFile(os.path.join(two, "model.safetensors")) as y, \
            SafetensorsFile(os.path.join(three, "model.safetensors")) as z:
        name = "model.layers.2.conv.in_proj.weight"
        assert torch.equal(x.tensor(name), y.tensor(name)) and not torch.equal(x.tensor(name), z.tensor(name))
        norm = x.tensor("model.layers.2.ffn_norm.weight")
        assert norm.dtype == torch.float32 and 0.9 <= float(norm.min()) and float(norm.max()) <= 1.1
        assert x.tensor(name).dtype == torch.bfloat16 and abs(float(x.tensor(name).float().std()) - 0.02) < 0.002
    with open(os.path.join(one, "config.json")) as handle:
        assert json.load(handle)["architectures"] == ["Lfm2ForCausalLM"]


def test_no_files(tmp_path):
    with pytest.raises(SafetensorsError, match="no .safetensors"):
        load_tensors(str(tmp_path), {}, torch.float32, CPU)
