"""The safetensors reader and writer, binding by name, the one error that lists everything,
and the seeded random-weights mode."""

import json
import os
import struct

import pytest
import torch

import beholdd
from beholdd.weights import (SafetensorsError, SafetensorsReader, TensorSpec, WeightError, check_manifest,
                             random_tensor, stored_dtype, write_safetensors)


def raw_file(path, header, data=b""):
    blob = json.dumps(header).encode()
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)) + blob + data)


def test_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int64),
               "d": torch.randn(2, 2, 2).to(torch.float16), "e": torch.zeros(0, 4)}
    path = str(tmp_path / "m.safetensors")
    write_safetensors(path, tensors)
    reader = SafetensorsReader(path)
    assert sorted(reader.names()) == sorted(tensors)
    for name, value in tensors.items():
        assert torch.equal(reader.tensor(name), value) and reader.tensor(name).dtype == value.dtype
    from safetensors import safe_open
    with safe_open(path, framework="pt") as other:
        for name, value in tensors.items():
            assert torch.equal(other.get_tensor(name), value)
    reader.close()


def test_malformed_files_are_refused(tmp_path):
    p = str(tmp_path / "x.safetensors")
    cases = [
        (lambda: open(p, "wb").write(b"\x01\x02"), "shorter"),
        (lambda: open(p, "wb").write(struct.pack("<Q", 0)), "header length"),
        (lambda: open(p, "wb").write(struct.pack("<Q", 1 << 40)), "header length"),
        (lambda: open(p, "wb").write(struct.pack("<Q", 100) + b"{}"), "past the end"),
        (lambda: open(p, "wb").write(struct.pack("<Q", 2) + b"[]"), "JSON object"),
        (lambda: raw_file(p, {"t": {"dtype": "F64", "shape": [1], "data_offsets": [0, 8]}}, b"\0" * 8), "dtype"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}}, b"\0" * 4), "shape"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [4, 0]}}, b"\0" * 4), "reversed"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 4), "needs 8 bytes"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4), "ends at byte"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 6), "trailing"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [2, 6]}}, b"\0" * 6), "unused bytes"),
        (lambda: raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]},
                              "u": {"dtype": "F32", "shape": [1], "data_offsets": [2, 6]}}, b"\0" * 6), "overlaps"),
    ]
    for make, message in cases:
        make()
        with pytest.raises(SafetensorsError, match=message):
            SafetensorsReader(p)
    raw_file(p, {"__metadata__": {"format": "pt"}, "t": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 4)
    assert SafetensorsReader(p).names() == ["t"]


def test_shards_of_a_folder_and_duplicate_names(tmp_path):
    write_safetensors(str(tmp_path / "model-00002.safetensors"), {"b": torch.ones(2)})
    write_safetensors(str(tmp_path / "model-00001.safetensors"), {"a": torch.zeros(2)})
    reader = SafetensorsReader(str(tmp_path))
    assert [os.path.basename(f) for f in reader.files] == ["model-00001.safetensors", "model-00002.safetensors"]
    assert sorted(reader.names()) == ["a", "b"]
    write_safetensors(str(tmp_path / "model-00003.safetensors"), {"a": torch.zeros(2)})
    with pytest.raises(SafetensorsError, match="occurs in both"):
        SafetensorsReader(str(tmp_path))
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(SafetensorsError, match="no .safetensors"):
        SafetensorsReader(str(empty))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path, model_dirs, tiny_configs):
    folder = model_dirs("B", "float32")
    reader = SafetensorsReader(folder)
    tensors = {name: reader.tensor(name).clone() for name in reader.names()}
    reader.close()
    del tensors["model.layers.1.self_attn.q_norm.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(256)
    tensors["model.layers.03.mlp.up_proj.weight"] = torch.zeros(160, 96)
    tensors["model.layers.2.mlp.down_proj.weight"] = torch.zeros(160, 96)       # transposed
    tensors["model.norm.weight"] = torch.zeros(96, dtype=torch.int32)
    broken = tmp_path / "broken"
    broken.mkdir()
    (broken / "config.json").write_text(json.dumps(tiny_configs["B"]))
    write_safetensors(str(broken / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as caught:
        beholdd.load_model(str(broken), "float32", "cpu")
    error = caught.value
    assert error.missing == ["model.layers.1.self_attn.q_norm.weight", "lm_head.weight"]
    assert sorted(error.unexpected) == ["model.layers.0.self_attn.q_proj.bias", "model.layers.03.mlp.up_proj.weight"]
    text = str(error)
    assert "model.layers.2.mlp.down_proj.weight: expected shape [96, 160], checkpoint has [160, 96]" in text
    assert "model.norm.weight: expected a float tensor, checkpoint has dtype I32" in text
    assert "missing tensors (2)" in text and "unexpected tensors (2)" in text


def test_tied_and_untied_heads_must_agree_with_the_file(tmp_path, model_dirs, tiny_configs):
    folder = model_dirs("B", "float32")        # untied: has lm_head.weight
    tied = tmp_path / "tied"
    tied.mkdir()
    (tied / "config.json").write_text(json.dumps(dict(tiny_configs["B"], tie_word_embeddings=True)))
    os.symlink(os.path.join(folder, "model.safetensors"), tied / "model.safetensors")
    with pytest.raises(WeightError, match="unexpected tensors .1.: lm_head.weight"):
        beholdd.load_model(str(tied), "float32", "cpu")


def test_storage_rule():
    bf16, f32 = torch.bfloat16, torch.float32
    assert stored_dtype(bf16, bf16) == bf16 and stored_dtype(torch.float16, bf16) == bf16
    assert stored_dtype(f32, bf16) == f32                       # stored in 32-bit: stays so
    assert stored_dtype(bf16, f32) == f32 and stored_dtype(f32, f32) == f32
    assert stored_dtype(torch.int64, bf16) == torch.int32 and stored_dtype(torch.int32, f32) == torch.int32


def test_random_weights_depend_on_seed_and_name_only(tmp_path, tiny_configs):
    spec = TensorSpec("model.layers.0.mlp.up_proj.weight", (40, 30), "linear")
    norm = TensorSpec("model.norm.weight", (500,), "norm")
    assert torch.equal(random_tensor(spec, 1), random_tensor(spec, 1))
    assert not torch.equal(random_tensor(spec, 1), random_tensor(spec, 2))
    assert not torch.equal(random_tensor(spec, 1), random_tensor(TensorSpec("other", (40, 30)), 1))
    big = random_tensor(TensorSpec("w", (400, 400)), 0)
    assert abs(float(big.std()) - 0.02) < 0.001 and abs(float(big.mean())) < 0.001
    assert abs(float(random_tensor(norm, 0).mean()) - 1.0) < 0.005
    a = beholdd.write_random_model(str(tmp_path / "a"), tiny_configs["A"], seed=3, dtype="bfloat16")
    b = beholdd.write_random_model(str(tmp_path / "b"), tiny_configs["A"], seed=3, dtype="float32")
    ra, rb = SafetensorsReader(a), SafetensorsReader(b)
    assert sorted(os.listdir(a)) == ["config.json", "model.safetensors"]
    assert len(ra.names()) == 24 and sum(ra.tensor(n).numel() for n in ra.names()) == 90496
    for name in ra.names():
        assert ra.entries[name].dtype == "BF16" and rb.entries[name].dtype == "F32"
        assert torch.equal(ra.tensor(name), rb.tensor(name).to(torch.bfloat16))      # round to nearest even
    assert json.load(open(os.path.join(a, "config.json"))) == tiny_configs["A"]
    check_manifest(beholdd.resolve_architecture(tiny_configs["A"]).build(
        beholdd.Qwen3Config.from_dict(tiny_configs["A"])).tensor_specs(), ra)
