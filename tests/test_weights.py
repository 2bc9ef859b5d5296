"""Safetensors reading and writing, binding by name and its one error, random weights. No GPU."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from tiny import TINY_A, TINY_B
from microllm_rocm_amd.architectures.qwen2 import build_spec
from microllm_rocm_amd.parts import INT_TABLE, MATRIX, Model, Runtime, TensorDecl, VECTOR
from microllm_rocm_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, load_folder, save_file,
                                       write_model_folder)
from microllm_rocm_amd.weights.loader import place, placed_dtype

CPU = torch.device("cpu")


def _decls(config, dtype=torch.float32):
    return Model(build_spec(config), Runtime(dtype=dtype, device=CPU)).tensors()


def test_round_trip_all_dtypes(tmp_path):
    tensors = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3),
               "b": torch.randn(5, 4).to(torch.bfloat16), "c": torch.randn(7).to(torch.float16),
               "d": torch.arange(4, dtype=torch.int32), "e": torch.zeros((0, 3))}
    path = str(tmp_path / "x.safetensors")
    save_file(tensors, path, metadata={"format": "pt"})
    handle = SafetensorsFile(path)
    assert handle.names() == list(tensors)
    for name, tensor in tensors.items():
        loaded = handle.tensor(name)
        assert loaded.dtype == tensor.dtype and loaded.shape == tensor.shape and torch.equal(loaded, tensor)
    handle.close()
    # the plain reader, which shares no code, reads the same numbers
    del tensors["d"]
    path = str(tmp_path / "floats.safetensors")
    save_file(tensors, path)
    independent = plain.read_safetensors(path)
    for name, tensor in tensors.items():
        np.testing.assert_array_equal(independent[name], tensor.to(torch.float64).numpy())


def test_official_package_reads_our_file_and_we_read_theirs(tmp_path):
    safetensors_torch = pytest.importorskip("safetensors.torch")
    tensors = {"w": torch.randn(3, 5).to(torch.bfloat16), "v": torch.randn(4)}
    ours = str(tmp_path / "ours.safetensors")
    save_file(tensors, ours)
    theirs = safetensors_torch.load_file(ours)
    assert all(torch.equal(theirs[name], tensors[name]) for name in tensors)
    other = str(tmp_path / "theirs.safetensors")
    safetensors_torch.save_file(tensors, other)
    handle = SafetensorsFile(other)
    assert all(torch.equal(handle.tensor(name), tensors[name]) for name in tensors)


def _write_raw(path, header: dict, payload: bytes):
    raw = json.dumps(header).encode()
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw)) + raw + payload)


@pytest.mark.parametrize("header,payload,text", [
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 12, "no tensor owns"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12, "hole"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
      "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12, "overlap"),
    ({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, "needs 12"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 16]}}, b"\0" * 8, "outside the payload"),
    ({"a": {"dtype": "Q4", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, "unsupported dtype"),
    ({"a": {"dtype": "F32", "shape": [-2], "data_offsets": [0, 8]}}, b"\0" * 8, "bad shape"),
])
def test_corrupt_files_are_refused(tmp_path, header, payload, text):
    # the negative cases of tests/io/safetensors_test.cpp:129-178
    path = str(tmp_path / "bad.safetensors")
    _write_raw(path, header, payload)
    with pytest.raises(SafetensorsError, match=text):
        SafetensorsFile(path)


def test_bad_header_length_and_shards(tmp_path):
    path = str(tmp_path / "short.safetensors")
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(path)
    folder = tmp_path / "sharded"
    folder.mkdir()
    save_file({"a": torch.ones(2)}, str(folder / "s1.safetensors"))
    save_file({"b": torch.ones(3)}, str(folder / "s2.safetensors"))
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    decls = {"a": TensorDecl((2,), VECTOR), "b": TensorDecl((3,), VECTOR)}
    loaded = load_folder(str(folder), decls, torch.float32, CPU)
    assert loaded["a"].shape == (2,) and loaded["b"].shape == (3,)
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "../s1.safetensors"}}))
    with pytest.raises(SafetensorsError, match="inside the folder"):
        load_folder(str(folder), decls, torch.float32, CPU)
    save_file({"a": torch.ones(2)}, str(folder / "s2.safetensors"))
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    with pytest.raises(SafetensorsError, match="both"):
        load_folder(str(folder), decls, torch.float32, CPU)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_model_folder(str(tmp_path / "m"), TINY_B, seed=1)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {name: handle.tensor(name).clone() for name in handle.names()}
    del tensors["model.layers.1.self_attn.k_proj.bias"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.extra.weight"] = torch.zeros(2, 2)
    tensors["model.layers.2.mlp.down_proj.weight"] = torch.zeros(96, 255)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as caught:
        load_folder(folder, _decls(TINY_B), torch.float32, CPU)
    error = caught.value
    assert error.missing == ["model.layers.1.self_attn.k_proj.bias", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.mlp.extra.weight"]
    assert len(error.incompatible) == 1 and "source=[96, 255] target=[96, 256]" in error.incompatible[0]
    text = str(error)
    assert "missing: model.norm.weight" in text and "unexpected: model.layers.0.mlp.extra.weight" in text


def test_tied_head_refuses_a_head_tensor(tmp_path):
    # tests/model/weights_test.cpp:217-221: a tied model binds no lm_head.weight
    folder = write_model_folder(str(tmp_path / "a"), TINY_A, seed=0)
    assert "lm_head.weight" not in _decls(TINY_A)
    handle = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {name: handle.tensor(name).clone() for name in handle.names()}
    tensors["lm_head.weight"] = torch.zeros(256, 64)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError, match="unexpected: lm_head.weight"):
        load_folder(folder, _decls(TINY_A), torch.float32, CPU)


def test_dtype_placement():
    matrix, vector, table = TensorDecl((2, 2), MATRIX), TensorDecl((2,), VECTOR), TensorDecl((2,), INT_TABLE)
    assert placed_dtype(torch.bfloat16, matrix, torch.bfloat16) == torch.bfloat16   # kept in bfloat16
    assert placed_dtype(torch.float32, matrix, torch.bfloat16) == torch.float32     # stored in 32-bit: stays so
    assert placed_dtype(torch.bfloat16, matrix, torch.float32) == torch.float32     # the 32-bit engine widens
    assert placed_dtype(torch.float16, matrix, torch.bfloat16) == torch.float32
    assert placed_dtype(torch.bfloat16, vector, torch.bfloat16) == torch.float32
    assert placed_dtype(torch.int64, table, torch.bfloat16) == torch.int32
    value = torch.tensor([1.0, 2.5]).to(torch.bfloat16)
    assert torch.equal(place(value, vector, torch.bfloat16, CPU), torch.tensor([1.0, 2.5]))


def test_random_folder_is_seeded_and_follows_the_rules(tmp_path):
    first = write_model_folder(str(tmp_path / "one"), TINY_B, seed=2, stds={"std": 0.02, "norm_std": 0.1})
    second = write_model_folder(str(tmp_path / "two"), TINY_B, seed=2, stds={"std": 0.02, "norm_std": 0.1})
    third = write_model_folder(str(tmp_path / "three"), TINY_B, seed=3, stds={"std": 0.02, "norm_std": 0.1})
    a, b, c = (plain.read_safetensors(os.path.join(f, "model.safetensors")) for f in (first, second, third))
    assert set(a) == set(_decls(TINY_B)) and all(np.array_equal(a[name], b[name]) for name in a)
    assert not np.array_equal(a["lm_head.weight"], c["lm_head.weight"])
    assert abs(a["model.embed_tokens.weight"].std() - 0.02) < 2e-3
    assert abs(a["model.layers.0.self_attn.q_proj.bias"].std() - 0.02) < 6e-3
    norm = a["model.layers.1.input_layernorm.weight"]
    assert abs(norm.mean() - 1.0) < 0.05 and 0.05 < norm.std() < 0.15
    plain_config = plain.read_config(first)
    assert plain_config["sliding_window"] == 24 and plain_config["max_window_layers"] == 1
    ones = plain.read_safetensors(os.path.join(write_model_folder(str(tmp_path / "a"), TINY_A, seed=0), "model.safetensors"))
    assert np.all(ones["model.norm.weight"] == 1.0)


def test_model_folder_command(tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    TINY_A.save(str(tmp_path / "src"))
    out = tmp_path / "made"
    result = subprocess.run([sys.executable, os.path.join(root, "bin", "microllm_make_model"), "--config", str(tmp_path / "src"),
                             "--seed", "4", "--out", str(out), "--std", "0.05"], capture_output=True, text=True)
    assert result.returncode == 0, result.stderr
    weights = plain.read_safetensors(str(out / "model.safetensors"))
    assert set(weights) == set(_decls(TINY_A)) and abs(weights["model.embed_tokens.weight"].std() - 0.05) < 5e-3
    assert plain.read_config(str(out))["hidden_size"] == 64
