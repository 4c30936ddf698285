"""Configuration, registry and engine options (no GPU)."""

from __future__ import annotations

import json

import pytest
from helpers import tiny_a, tiny_b

from miniserve_amd.config import (
    ConfigError,
    EngineConfig,
    Qwen3Config,
    config_from_dict,
    load_config,
    register_architecture,
    registered_architectures,
)


def qwen3_0_6b() -> dict:
    # the dict of the reference's own test (tests/unit/test_config.py:14-34)
    return {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_size": 1024,
        "intermediate_size": 3072,
        "num_hidden_layers": 28,
        "num_attention_heads": 16,
        "num_key_value_heads": 8,
        "head_dim": 128,
        "rms_norm_eps": 1e-6,
        "rope_theta": 1_000_000,
        "max_position_embeddings": 40_960,
        "vocab_size": 151_936,
        "hidden_act": "silu",
        "attention_bias": False,
        "attention_dropout": 0.0,
        "tie_word_embeddings": True,
        "sliding_window": None,
        "use_sliding_window": False,
    }


def test_head_dim_is_read_not_derived():
    # reference: tests/unit/test_config.py:83-86 (128, not 1024 / 16 = 64)
    config = config_from_dict(qwen3_0_6b())
    assert isinstance(config, Qwen3Config)
    assert config.head_dim == 128 and config.hidden_size // config.num_attention_heads == 64
    spec = config.model_spec()
    attention = spec.layers[0].mixer
    assert attention.params["head_dim"] == 128 and attention.params["num_kv_heads"] == 8
    assert attention.params["scale"] == 128**-0.5
    assert attention.params["position"].params == {"dim": 128, "theta": 1_000_000.0}
    assert len(spec.layers) == 28 and [c.layer for c in spec.order] == list(range(28))
    assert spec.head.params["tied_to"] == "model.embed_tokens.weight"


def test_untied_head_is_accepted_and_round_trips():
    config = config_from_dict(tiny_b())
    assert config.tie_word_embeddings is False
    assert config.model_spec().head.params["tied_to"] is None
    again = config_from_dict(json.loads(json.dumps(config.to_dict())))
    assert again == config


def test_no_size_stands_in_code():
    a, b = config_from_dict(tiny_a()).model_spec(), config_from_dict(tiny_b()).model_spec()
    for spec, source in ((a, tiny_a()), (b, tiny_b())):
        mixer, ffn = spec.layers[0].mixer.params, spec.layers[0].feed_forward.params
        assert mixer["num_heads"] == source["num_attention_heads"]
        assert mixer["q_norm"].params["eps"] == source["rms_norm_eps"]
        assert mixer["q_norm"].params["dim"] == source["head_dim"]
        assert ffn["intermediate_size"] == source["intermediate_size"]
        assert spec.final_norm.params["dim"] == source["hidden_size"]
        assert spec.vocab_size == source["vocab_size"]


@pytest.mark.parametrize(
    ("override", "message"),
    [
        # reference: tests/unit/test_config.py:113-152
        ({"model_type": "llama"}, "UNSUPPORTED_MODEL_CONFIGURATION"),
        ({"sliding_window": 4096}, "Sliding-window"),
        ({"use_sliding_window": True}, "Sliding-window"),
        ({"rope_scaling": {"rope_type": "linear", "factor": 2.0}}, "scaled RoPE"),
        ({"rope_interleaved": True}, "Interleaved"),
        ({"attention_bias": True}, "bias-free"),
        ({"mlp_bias": True}, "bias-free"),
        ({"attention_dropout": 0.1}, "dropout-free"),
        ({"hidden_act": "gelu"}, "SiLU"),
        ({"num_key_value_heads": 3}, "divisible"),
        ({"head_dim": 127}, "even head_dim"),
        ({"hidden_size": 1024.5}, "hidden_size must be an integer"),
        ({"num_attention_heads": True}, "num_attention_heads must be an integer"),
        ({"head_dim": "128"}, "head_dim must be an integer"),
        ({"rms_norm_eps": float("nan")}, "finite and positive"),
        ({"rope_theta": float("inf")}, "finite and positive"),
        ({"rope_theta": 0}, "finite and positive"),
        ({"tie_word_embeddings": 1}, "tie_word_embeddings must be boolean"),
        ({"attention_dropout": "0.0"}, "attention_dropout must be numeric"),
        ({"vocab_size": 0}, "vocab_size must be positive"),
        ({"architectures": ["A", "B"]}, "exactly one"),
    ],
)
def test_rejected_variants(override, message):
    data = qwen3_0_6b()
    data.update(override)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(data)


def test_missing_head_dim_is_an_error():
    data = qwen3_0_6b()
    del data["head_dim"]
    with pytest.raises(ConfigError, match="head_dim"):
        config_from_dict(data)


def test_registry_names_unknown_architectures():
    data = qwen3_0_6b()
    data["architectures"] = ["SomethingElseForCausalLM"]
    with pytest.raises(ConfigError, match="UNSUPPORTED_MODEL_CONFIGURATION.*SomethingElse"):
        config_from_dict(data)
    assert "Qwen3ForCausalLM" in registered_architectures()
    with pytest.raises(TypeError):
        register_architecture("Broken", object)


def test_load_config_reads_the_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(tiny_a()))
    assert load_config(tmp_path).vocab_size == 256
    with pytest.raises(FileNotFoundError):
        load_config(tmp_path / "nowhere")


def test_engine_config_rules():
    # reference: engine_config.py:288-291, runtime_config.py:85-86, model_config.py:204-205
    EngineConfig().validate(max_positions=512)
    with pytest.raises(ConfigError, match="position limit"):
        EngineConfig(max_model_len=1024).validate(max_positions=512)
    with pytest.raises(ConfigError, match="requires enable_chunked_prefill"):
        EngineConfig(prefill_chunk_size=8).validate(max_positions=512)
    with pytest.raises(ConfigError, match="cannot exceed max_num_batched_tokens"):
        EngineConfig(enable_chunked_prefill=True, prefill_chunk_size=64, max_num_batched_tokens=32).validate(
            max_positions=512
        )
    with pytest.raises(ConfigError, match="cannot exceed max_model_len"):
        EngineConfig(max_num_batched_tokens=1024).validate(max_positions=512)
    with pytest.raises(ConfigError, match="dtype"):
        EngineConfig(dtype="float16").validate(max_positions=512)
    for name, value in (("max_num_seqs", True), ("kv_block_size", 1.5), ("num_kv_blocks", 2.5), ("max_model_len", 0)):
        with pytest.raises(ConfigError, match=name):
            EngineConfig(**{name: value}).validate(max_positions=512)
    assert EngineConfig().resolved_max_num_batched_tokens(512) == 512
    assert EngineConfig().resolved_max_num_batched_tokens(40960) == 4096


def test_presets_are_config_files_of_registered_architectures(tmp_path):
    from miniserve_amd.config import config_dict_from_preset_or_file, config_from_dict, preset_names

    assert preset_names() == ("qwen3-0.6b", "qwen3-32b", "qwen3-8b")
    for name in preset_names():
        config = config_from_dict(config_dict_from_preset_or_file(name.upper()))       # names in any case
        spec = config.model_spec()
        assert spec.vocab_size == 151936 and len(spec.layers) == config.num_hidden_layers
    small = config_from_dict(config_dict_from_preset_or_file("qwen3-0.6b"))
    assert (small.hidden_size, small.num_attention_heads, small.num_key_value_heads, small.tie_word_embeddings) == (1024, 16, 8, True)
    path = tmp_path / "config.json"
    path.write_text(json.dumps({**config_dict_from_preset_or_file("qwen3-8b"), "num_hidden_layers": 3}))
    assert config_from_dict(config_dict_from_preset_or_file(str(path))).num_hidden_layers == 3
    with pytest.raises(FileNotFoundError, match="neither a config.json nor one of the presets"):
        config_dict_from_preset_or_file("qwen3-7b")
