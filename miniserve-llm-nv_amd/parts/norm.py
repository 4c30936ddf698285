"""RMSNorm part (reference: miniserve/model/layers.py:10-34)."""

from __future__ import annotations

from typing import Mapping

import torch

from .. import ops
from ..config.model_spec import PartSpec
from .base import Part, WeightSpec, register_part, require_params


class RMSNorm(Part):
    """``y = w * round(x * rsqrt(mean(x^2) + eps))`` with 32-bit statistics; no
    mean subtraction, no bias, the weight is plain ``w``."""

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "dim", "eps")
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        if self.dim <= 0 or not self.eps > 0:
            raise ValueError("RMSNorm needs dim > 0 and eps > 0.")
        self.dtype = dtype
        self.weight_name = spec.prefix + "weight"
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.weight_name, (self.dim,), init="norm")]

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """``x [..., dim]`` of the part's dtype (or float32) -> the part's dtype."""

        flat = x.reshape(-1, self.dim)
        return ops.rmsnorm(flat, self.weight, self.eps).reshape(x.shape)

    def add_forward(
        self,
        residual: torch.Tensor,
        delta: torch.Tensor | None,
        *,
        rows: torch.Tensor | None = None,
        write_back: bool = True,
    ) -> torch.Tensor:
        """Norm of ``residual + delta`` (``residual`` float32 ``[N, dim]``); the sum
        is stored back unless ``rows`` selects output rows or ``write_back`` is off."""

        if delta is None:
            return ops.rmsnorm(residual, self.weight, self.eps, rows=rows)
        return ops.rmsnorm(
            residual, self.weight, self.eps, delta=delta, rows=rows, write_back=write_back and rows is None
        )


register_part("norm", "rmsnorm", RMSNorm)
