"""Typed configuration of the Qwen3 dense decoder, read from its ``config.json``.

Same keys, same no-coercion rule and same rejected variants as the reference
(reference: miniserve/config/model_config.py:60-215), with two differences that
this engine needs: ``tie_word_embeddings=false`` is accepted (an untied
``lm_head.weight``), and the compute dtype is an engine option, not a model one.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Any, Mapping

from .fields import (
    ConfigError,
    read_architecture,
    read_bool,
    read_finite_positive,
    read_number,
    read_positive_int,
    read_str,
)
from .model_spec import LayerCall, LayerSpec, ModelSpec, PartSpec
from .registry import register_architecture


@dataclass(frozen=True)
class Qwen3Config:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    attention_bias: bool = False
    attention_dropout: float = 0.0
    mlp_bias: bool = False

    architecture = "Qwen3ForCausalLM"
    model_type = "qwen3"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "Qwen3Config":
        """Read and check a ``config.json`` mapping.

        ``head_dim`` is read, never derived from ``hidden_size / heads``
        (Qwen3-0.6B: 128, not 64; reference: model_config.py:112-117).
        Unknown keys are ignored (reference: model_config.py:130-163)."""

        architecture = read_architecture(data)
        model_type = data.get("model_type")
        if architecture != cls.architecture or model_type != cls.model_type:
            raise ConfigError(
                "UNSUPPORTED_MODEL_CONFIGURATION: expected architectures=['Qwen3ForCausalLM'] "
                f"with model_type='qwen3', got {architecture!r} / {model_type!r}."
            )
        if "head_dim" not in data:
            raise ConfigError("Qwen3 model config must define integer head_dim.")
        config = cls(
            hidden_size=read_positive_int(data, "hidden_size"),
            intermediate_size=read_positive_int(data, "intermediate_size"),
            num_hidden_layers=read_positive_int(data, "num_hidden_layers"),
            num_attention_heads=read_positive_int(data, "num_attention_heads"),
            num_key_value_heads=read_positive_int(data, "num_key_value_heads"),
            head_dim=read_positive_int(data, "head_dim"),
            vocab_size=read_positive_int(data, "vocab_size"),
            max_position_embeddings=read_positive_int(data, "max_position_embeddings"),
            rms_norm_eps=read_finite_positive(data, "rms_norm_eps"),
            rope_theta=read_finite_positive(data, "rope_theta"),
            tie_word_embeddings=read_bool(data, "tie_word_embeddings", False),
            hidden_act=read_str(data, "hidden_act", ""),
            attention_bias=read_bool(data, "attention_bias", False),
            attention_dropout=read_number(data, "attention_dropout"),
            mlp_bias=read_bool(data, "mlp_bias", False),
        )
        # Variants that the reference rejects (model_config.py:206-213) and this
        # engine does not run either.
        if read_bool(data, "rope_interleaved", False) or data.get("rope_scaling") is not None:
            raise ConfigError("Interleaved or scaled RoPE is not implemented.")
        if data.get("sliding_window") is not None or read_bool(data, "use_sliding_window", False):
            raise ConfigError("Sliding-window attention is not implemented for Qwen3.")
        config.validate()
        return config

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("num_attention_heads must be divisible by num_key_value_heads.")
        if self.head_dim % 2 != 0:
            raise ConfigError("RoPE requires an even head_dim.")
        if self.hidden_act != "silu":
            raise ConfigError("Only the Qwen3 SiLU MLP is implemented.")
        if self.attention_bias or self.attention_dropout != 0.0 or self.mlp_bias:
            raise ConfigError("Only bias-free, dropout-free dense attention/MLP is implemented.")

    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` mapping that :meth:`from_dict` reads back."""

        data: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
        }
        data.update(asdict(self))
        data.update(
            rope_scaling=None,
            sliding_window=None,
            use_sliding_window=False,
        )
        return data

    def model_spec(self) -> ModelSpec:
        """Qwen3 as parts: every layer is the same pre-norm block of a GQA
        attention (per-head q/k RMSNorm, half-split rotary) and a gated SiLU
        MLP (reference: miniserve/model/qwen3.py:326-347, layers.py:71-87)."""

        def rmsnorm(dim: int, prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", {"dim": dim, "eps": self.rms_norm_eps}, prefix)

        layers = []
        for index in range(self.num_hidden_layers):
            base = f"model.layers.{index}."
            attention = PartSpec(
                "attention",
                {
                    "hidden_size": self.hidden_size,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    # reference: qwen3.py:66, scaling = head_dim ** -0.5
                    "scale": self.head_dim**-0.5,
                    "window": None,
                    "q_norm": rmsnorm(self.head_dim, base + "self_attn.q_norm."),
                    "k_norm": rmsnorm(self.head_dim, base + "self_attn.k_norm."),
                    "position": PartSpec("rotary_half", {"dim": self.head_dim, "theta": self.rope_theta}),
                },
                base + "self_attn.",
            )
            mlp = PartSpec(
                "gated_mlp",
                {
                    "hidden_size": self.hidden_size,
                    "intermediate_size": self.intermediate_size,
                    "activation": self.hidden_act,
                },
                base + "mlp.",
            )
            layers.append(
                LayerSpec(
                    block="prenorm",
                    mixer=attention,
                    feed_forward=mlp,
                    norms={
                        "pre_mixer": rmsnorm(self.hidden_size, base + "input_layernorm."),
                        "pre_feed_forward": rmsnorm(self.hidden_size, base + "post_attention_layernorm."),
                    },
                )
            )
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec(
                "token_embedding",
                {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size},
                "model.embed_tokens.",
            ),
            layers=tuple(layers),
            order=tuple(LayerCall(index) for index in range(self.num_hidden_layers)),
            final_norm=rmsnorm(self.hidden_size, "model.norm."),
            head=PartSpec(
                "linear_head",
                {
                    "vocab_size": self.vocab_size,
                    "hidden_size": self.hidden_size,
                    "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None,
                },
                "lm_head.",
            ),
        )


register_architecture(Qwen3Config.architecture, Qwen3Config)
