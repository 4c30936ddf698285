"""Token embedding and the output head (reference: miniserve/model/qwen3.py:413,534-540,558)."""

from __future__ import annotations

from typing import Mapping

import torch

from .. import ops
from ..config.model_spec import PartSpec
from .base import Part, WeightSpec, register_part, require_params


class TokenEmbedding(Part):
    """``h[t] = E[token_id[t]]``: a row gather, no scaling, no position term."""

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "vocab_size", "hidden_size")
        self.vocab_size = int(params["vocab_size"])
        self.hidden_size = int(params["hidden_size"])
        self.weight_name = spec.prefix + "weight"
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.weight_name, (self.vocab_size, self.hidden_size))]

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name]

    def forward(self, token_ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """``ctx``: the step's context, which every embedding part is handed (one that
        adds a term of the position reads it there); this one needs the ids alone."""

        return ops.embedding_gather(token_ids, self.weight)


class LinearHead(Part):
    """``logits = y W^T`` without bias, soft-cap or scaling, as float32.  Tied:
    ``W`` is the embedding tensor itself and ``<prefix>weight`` is optional in
    the checkpoint but must equal it when present (reference: loader.py:132-152)."""

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "vocab_size", "hidden_size")
        self.vocab_size = int(params["vocab_size"])
        self.hidden_size = int(params["hidden_size"])
        self.tied_to = params.get("tied_to")
        self.weight_name = spec.prefix + "weight"
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        shape = (self.vocab_size, self.hidden_size)
        if self.tied_to:
            return [WeightSpec(self.weight_name, shape, optional=True, same_as=self.tied_to)]
        return [WeightSpec(self.weight_name, shape)]

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tied_to] if self.tied_to else tensors[self.weight_name]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(x, self.weight, out_float32=True)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
