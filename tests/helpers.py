"""Shared test material: the tiny configurations, model folders with random
weights in a temporary place, and replay shapes."""

from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def tiny_a() -> dict:
    """2 layers, hidden 64, 4 q heads, 2 kv heads, head 16, inter 128, vocab 256,
    theta 1e4, eps 1e-6, tied; pages of 16."""

    return {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_size": 64,
        "intermediate_size": 128,
        "num_hidden_layers": 2,
        "num_attention_heads": 4,
        "num_key_value_heads": 2,
        "head_dim": 16,
        "vocab_size": 256,
        "max_position_embeddings": 512,
        "rms_norm_eps": 1e-6,
        "rope_theta": 10000.0,
        "tie_word_embeddings": True,
        "hidden_act": "silu",
        "attention_bias": False,
        "attention_dropout": 0.0,
    }


def tiny_b() -> dict:
    """Differs from A in every size and option: 3 layers, hidden 96, 8 q heads, 1 kv
    head (group 8), head 32 (q width 256 != hidden), inter 200, vocab 509, theta
    1e6, eps 1e-5, untied head; pages of 8."""

    return {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_size": 96,
        "intermediate_size": 200,
        "num_hidden_layers": 3,
        "num_attention_heads": 8,
        "num_key_value_heads": 1,
        "head_dim": 32,
        "vocab_size": 509,
        "max_position_embeddings": 1024,
        "rms_norm_eps": 1e-5,
        "rope_theta": 1000000.0,
        "tie_word_embeddings": False,
        "hidden_act": "silu",
        "attention_bias": False,
        "attention_dropout": 0.0,
    }


def tiny_c() -> dict:
    """A third one with wider heads and larger pages, and a group of three query heads
    to a kv head: 2 layers, hidden 80,
    6 q heads, 2 kv heads (group 3), head 64, inter 176, vocab 300, theta 5e5, eps
    1e-6, untied head; pages of 32."""

    return {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_size": 80,
        "intermediate_size": 176,
        "num_hidden_layers": 2,
        "num_attention_heads": 6,
        "num_key_value_heads": 2,
        "head_dim": 64,
        "vocab_size": 300,
        "max_position_embeddings": 1024,
        "rms_norm_eps": 1e-6,
        "rope_theta": 500000.0,
        "tie_word_embeddings": False,
        "hidden_act": "silu",
        "attention_bias": False,
        "attention_dropout": 0.0,
    }


TINY = {"a": (tiny_a, 16), "b": (tiny_b, 8), "c": (tiny_c, 32)}


def make_model_folder(folder: Path, config_dict: dict, seed: int, store_dtype: str = "float32") -> Path:
    from miniserve_amd.config import config_from_dict
    from miniserve_amd.weights import write_random_model

    return write_random_model(config_from_dict(config_dict), folder, seed=seed, store_dtype=store_dtype)


def read_weights(folder: Path) -> dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(str(Path(folder) / "model.safetensors"))


def read_config(folder: Path) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def random_tokens(length: int, vocab: int, seed: int) -> list[int]:
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=generator).tolist()
