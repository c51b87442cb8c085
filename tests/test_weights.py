"""Weights: the safetensors reader and writer, loading by name, the one error
that lists everything, the kept types, the random-weights folder."""

import json
import struct

import pytest
import torch

import tiny_models
from rvllm_amd.models import DecoderModel, load_config
from rvllm_amd.parts.base import ParamSpec
from rvllm_amd.models.gemma3 import locate_tensors
from rvllm_amd.weights.loader import WeightError, load_tensors, open_model_files, tensor_names
from rvllm_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, resolve_shards, write_safetensors


def raw_file(path, header: dict, payload: bytes):
    text = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(text)) + text + payload)
    return path


def test_round_trip_matches_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {
        "a": torch.randn(3, 5).to(torch.bfloat16),
        "b": torch.arange(7, dtype=torch.int32),
        "c": torch.randn(2, 2, 2),
        "d": torch.randn(4).to(torch.float16),
    }
    write_safetensors(tmp_path / "ours.safetensors", tensors)
    theirs = load_file(str(tmp_path / "ours.safetensors"))  # the package reads what we write
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    f = SafetensorsFile(tmp_path / "theirs.safetensors")  # we read what the package writes
    for name, t in tensors.items():
        assert torch.equal(theirs[name], t)
        got = f.tensor(name)
        assert got.dtype == t.dtype and torch.equal(got, t)
    f.close()


def test_corrupt_files_are_refused(tmp_path):
    ok = {"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}
    SafetensorsFile(raw_file(tmp_path / "ok.st", ok, b"\0" * 8)).close()
    cases = {
        "short": (None, b"\x01"),
        "header too long": (None, struct.pack("<Q", 1000) + b"{}"),
        "not json": (None, struct.pack("<Q", 5) + b"{nope"),
        "bad dtype": ({"x": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}, b"\0" * 2),
        "size mismatch": ({"x": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8),
        "outside file": ({"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4),
        "overlap": ({"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
                     "y": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12),
        "negative dim": ({"x": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 0]}}, b""),
        "rank": ({"x": {"dtype": "F32", "shape": [1] * 17, "data_offsets": [0, 4]}}, b"\0" * 4),
    }
    for name, (header, payload) in cases.items():
        p = tmp_path / "bad.st"
        if header is None:
            p.write_bytes(payload)
        else:
            raw_file(p, header, payload)
        with pytest.raises(SafetensorsError):
            SafetensorsFile(p)
    # duplicate key in the header text
    text = b'{"x":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"x":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}}'
    (tmp_path / "dup.st").write_bytes(struct.pack("<Q", len(text)) + text + b"\0" * 4)
    with pytest.raises(SafetensorsError, match="duplicate"):
        SafetensorsFile(tmp_path / "dup.st")


def test_shard_index(tmp_path):
    write_safetensors(tmp_path / "m1.safetensors", {"a": torch.zeros(2)})
    write_safetensors(tmp_path / "m2.safetensors", {"b": torch.zeros(2)})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "m1.safetensors", "b": "m2.safetensors"}}))
    assert [p.name for p in resolve_shards(tmp_path)] == ["m1.safetensors", "m2.safetensors"]
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "../m1.safetensors"}}))
    with pytest.raises(SafetensorsError, match="leaves"):
        resolve_shards(tmp_path)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(SafetensorsError, match="neither"):
        resolve_shards(empty)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path, model_dirs):
    from safetensors.torch import load_file, save_file

    tensors = load_file(str(model_dirs["A"] / "model.safetensors"))
    del tensors["model.layers.0.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.extra.weight"] = torch.zeros(3)
    tensors["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(64, 63, dtype=torch.bfloat16)
    (tmp_path / "config.json").write_text((model_dirs["A"] / "config.json").read_text())
    save_file(tensors, str(tmp_path / "model.safetensors"))
    arch, cfg = load_config(tmp_path)
    files = open_model_files(tmp_path)
    model = DecoderModel(arch.build_spec(cfg, **arch.locate_tensors(tensor_names(files))))
    with pytest.raises(WeightError) as e:
        load_tensors(files, model.param_specs(), torch.bfloat16, source=str(tmp_path))
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.mlp.extra.weight"]
    assert err.wrong_shape == [("model.layers.1.self_attn.q_proj.weight", (64, 64), (64, 63))]
    text = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (1)", "expected [64, 64], got [64, 63]"):
        assert needle in text


def test_kept_types(tmp_path):
    write_safetensors(tmp_path / "model.safetensors", {
        "half": torch.ones(2, dtype=torch.float16),
        "brain": torch.ones(2, dtype=torch.bfloat16),
        "single": torch.full((2,), 1.0 + 2 ** -20, dtype=torch.float32),
        "table": torch.arange(3, dtype=torch.int64),
    })
    specs = [ParamSpec("half", (2,)), ParamSpec("brain", (2,)), ParamSpec("single", (2,)),
             ParamSpec("table", (3,), integer=True)]
    files = open_model_files(tmp_path)
    got = load_tensors(files, specs, torch.bfloat16)
    assert got["half"].dtype == torch.bfloat16 and got["brain"].dtype == torch.bfloat16
    assert got["single"].dtype == torch.float32 and got["single"][0].item() == 1.0 + 2 ** -20  # stays 32-bit
    assert got["table"].dtype == torch.int32
    got = load_tensors(files, specs, torch.float32)
    assert all(got[n].dtype == torch.float32 for n in ("half", "brain", "single"))
    assert got["table"].dtype == torch.int32
    # an integer where floats are expected is an error, not a cast
    with pytest.raises(WeightError, match="expected floating values"):
        load_tensors(files, [ParamSpec("table", (3,))] + specs[:3], torch.float32)


def test_prefix_detection():
    assert locate_tensors(["model.language_model.embed_tokens.weight"])["prefix"] == "model.language_model"
    assert locate_tensors(["language_model.model.embed_tokens.weight"])["prefix"] == "language_model.model"
    assert locate_tensors(["model.embed_tokens.weight", "x"]) == {"prefix": "model", "head_weight": "lm_head.weight"}


def test_an_untied_head_is_found_beside_a_nested_decoder():
    # as the reference looks it up: under no prefix (gemma4_load.rs:431-436)
    assert locate_tensors(["model.language_model.embed_tokens.weight", "lm_head.weight"])["head_weight"] == "lm_head.weight"
    # beside the decoder it belongs to
    assert locate_tensors(["language_model.model.embed_tokens.weight", "language_model.lm_head.weight"])[
        "head_weight"] == "language_model.lm_head.weight"
    assert locate_tensors(["language_model.embed_tokens.weight", "language_model.lm_head.weight"])[
        "head_weight"] == "language_model.lm_head.weight"
    # none there: the plain name, which the loader then reports missing
    assert locate_tensors(["model.embed_tokens.weight"])["head_weight"] == "lm_head.weight"


def test_nested_prefix_loads_and_ignores_the_vision_part(tmp_path, model_dirs):
    from safetensors.torch import load_file, save_file

    tensors = {k.replace("model.", "model.language_model.", 1): v
               for k, v in load_file(str(model_dirs["A"] / "model.safetensors")).items()}
    tensors["model.vision_tower.patch.weight"] = torch.zeros(2)
    (tmp_path / "config.json").write_text((model_dirs["A"] / "config.json").read_text())
    save_file(tensors, str(tmp_path / "model.safetensors"))
    arch, cfg = load_config(tmp_path)
    files = open_model_files(tmp_path)
    where = arch.locate_tensors(tensor_names(files))
    prefix = where["prefix"]
    model = DecoderModel(arch.build_spec(cfg, **where))
    got = load_tensors(files, model.param_specs(), torch.bfloat16, ignore=arch.ignored_prefixes)
    assert f"{prefix}.layers.1.mlp.down_proj.weight" in got and len(got) == 28


def test_random_model_folder_is_reproducible(tmp_path):
    a = tiny_models.write_model(tmp_path / "a", "B", seed=5)
    b = tiny_models.write_model(tmp_path / "b", "B", seed=5)
    c = tiny_models.write_model(tmp_path / "c", "B", seed=6)
    assert (a / "model.safetensors").read_bytes() == (b / "model.safetensors").read_bytes()
    assert (a / "model.safetensors").read_bytes() != (c / "model.safetensors").read_bytes()
    f = SafetensorsFile(a / "model.safetensors")
    emb = f.tensor("model.embed_tokens.weight").float()
    norm = f.tensor("model.layers.0.input_layernorm.weight").float()
    assert emb.shape == (509, 96) and abs(emb.std().item() - 0.02) < 0.002
    assert norm.shape == (96,) and 0.05 < norm.std().item() < 0.15  # zero-centred norm weights, N(0, 0.1)
    assert f.entries["model.embed_tokens.weight"].dtype_name == "BF16"
    f.close()
