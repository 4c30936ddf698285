"""Weights by tensor name: strict check, tied head, random-weights mode (no GPU)."""

from __future__ import annotations

import json

import pytest
import torch
from helpers import make_model_folder, read_weights, tiny_a, tiny_b
from safetensors.torch import save_file

from miniserve_amd.config import load_config
from miniserve_amd.parts import DecoderModel
from miniserve_amd.weights import WeightLoadError, load_weights, random_tensors


def specs_of(folder):
    return DecoderModel(load_config(folder).model_spec(), "float32").weight_specs()


def test_random_model_folder_loads_and_same_seed_same_model(tmp_path):
    first = make_model_folder(tmp_path / "one", tiny_b(), seed=5)
    second = make_model_folder(tmp_path / "two", tiny_b(), seed=5)
    other = make_model_folder(tmp_path / "three", tiny_b(), seed=6)
    a, b, c = read_weights(first), read_weights(second), read_weights(other)
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert any(not torch.equal(a[k], c[k]) for k in a)
    tensors, report = load_weights(first, specs_of(first), dtype=torch.float32, device="cpu")
    assert report.loaded_tensors == len(a) and set(tensors) == set(a)
    # expected names of the reference (miniserve/model/weight_map.py:19-45)
    assert "model.layers.2.self_attn.q_norm.weight" in tensors and "lm_head.weight" in tensors
    assert tensors["model.layers.0.self_attn.q_proj.weight"].shape == (8 * 32, 96)
    # distributions: matrices ~ N(0, 0.02), norm weights ~ 1 + N(0, 0.1)
    assert abs(float(a["model.embed_tokens.weight"].std()) - 0.02) < 0.002
    assert abs(float(a["model.layers.0.input_layernorm.weight"].mean()) - 1.0) < 0.05


def test_tied_model_stores_no_head_and_bfloat16_is_kept(tmp_path):
    folder = make_model_folder(tmp_path / "tied", tiny_a(), seed=1, store_dtype="bfloat16")
    stored = read_weights(folder)
    assert "lm_head.weight" not in stored
    tensors, report = load_weights(folder, specs_of(folder), dtype=torch.bfloat16, device="cpu")
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    assert report.source_dtype_counts == {"torch.bfloat16": len(stored)}


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_model_folder(tmp_path / "m", tiny_a(), seed=1)
    weights = read_weights(folder)
    del weights["model.norm.weight"]
    del weights["model.layers.1.mlp.up_proj.weight"]
    weights["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    weights["surprise.bias"] = torch.zeros(3)
    weights["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    weights["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(8)
    save_file(weights, str(folder / "model.safetensors"))
    with pytest.raises(WeightLoadError) as caught:
        load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")
    error = caught.value
    assert error.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.7.mlp.up_proj.weight", "surprise.bias"]
    assert [name for name, _, _ in error.wrong_shape] == [
        "model.layers.0.self_attn.k_proj.weight",
        "model.layers.0.self_attn.q_norm.weight",
    ]
    text = str(error)
    for needle in ("missing tensors (2)", "unexpected tensors (2)", "(16, 64)", "(32, 64)", "surprise.bias"):
        assert needle in text
    # a tensor of a layer that the model does not have is named as such (a checkpoint of a deeper model)
    assert "tensors of layers [7] are stored, the model has layers 0..1" in text


def test_init_rules_are_open(tmp_path):
    """A part names a rule that another package registered, or brings a callable."""

    from miniserve_amd.parts import WeightSpec
    from miniserve_amd.weights import register_init

    register_init("test_ones", lambda shape, generator, device: torch.ones(shape, dtype=torch.float32, device=device))
    specs = [
        WeightSpec("a", (2, 3), init="test_ones"),
        WeightSpec("b", (4,), init=lambda shape, generator, device: torch.full(shape, 7.0, device=device)),
        WeightSpec("c", (2, 2)),
    ]
    drawn = random_tensors(specs, seed=1)
    assert torch.equal(drawn["a"], torch.ones(2, 3)) and torch.equal(drawn["b"], torch.full((4,), 7.0))
    assert 0 < float(drawn["c"].abs().max()) < 0.2
    with pytest.raises(ValueError, match="unknown init rule"):
        random_tensors([WeightSpec("d", (1,), init="nobody")], seed=1)
    with pytest.raises(ValueError, match="float32 tensor of shape"):
        random_tensors([WeightSpec("e", (2,), init=lambda shape, generator, device: torch.zeros(3))], seed=1)


def test_tied_head_in_the_file_must_equal_the_embedding(tmp_path):
    folder = make_model_folder(tmp_path / "m", tiny_a(), seed=1)
    weights = read_weights(folder)
    weights["lm_head.weight"] = weights["model.embed_tokens.weight"].clone()
    save_file(weights, str(folder / "model.safetensors"))
    tensors, _ = load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")
    assert "lm_head.weight" not in tensors          # the embedding stands for both
    weights["lm_head.weight"][3, 4] += 1.0
    save_file(weights, str(folder / "model.safetensors"))
    with pytest.raises(WeightLoadError, match="tied to model.embed_tokens.weight but their values differ"):
        load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")


def test_shards_index_and_duplicates(tmp_path):
    folder = make_model_folder(tmp_path / "m", tiny_b(), seed=2)
    weights = read_weights(folder)
    (folder / "model.safetensors").unlink()
    names = sorted(weights)
    first, second = names[: len(names) // 2], names[len(names) // 2 :]
    save_file({n: weights[n] for n in first}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({n: weights[n] for n in second}, str(folder / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {n: "model-00001-of-00002.safetensors" for n in first}}
    index["weight_map"].update({n: "model-00002-of-00002.safetensors" for n in second})
    (folder / "model.safetensors.index.json").write_text(json.dumps(index))
    tensors, _ = load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")
    assert set(tensors) == set(weights)
    # a name in two shards (reference: loader.py:176-177)
    save_file({n: weights[n] for n in second + first[:1]}, str(folder / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightLoadError, match="duplicate tensor across shards"):
        load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")
    (folder / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(FileNotFoundError):
        load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")


def test_integer_tensor_where_a_float_is_wanted(tmp_path):
    folder = make_model_folder(tmp_path / "m", tiny_a(), seed=1)
    weights = read_weights(folder)
    weights["model.norm.weight"] = torch.ones(64, dtype=torch.int32)
    save_file(weights, str(folder / "model.safetensors"))
    with pytest.raises(WeightLoadError, match="floating type is wanted"):
        load_weights(folder, specs_of(folder), dtype=torch.float32, device="cpu")


def test_random_tensors_follow_spec_order():
    specs = DecoderModel(load_config_dict(tiny_a()).model_spec(), "float32").weight_specs()
    tensors = random_tensors(specs, seed=9)
    assert list(tensors) == [s.name for s in specs if s.same_as is None]


def load_config_dict(data):
    from miniserve_amd.config import config_from_dict

    return config_from_dict(data)
