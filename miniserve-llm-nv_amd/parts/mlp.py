"""Gated feed-forward: ``down(act(gate(x)) * up(x))``, no biases, every token the
same weights (reference: miniserve/model/layers.py:71-87)."""

from __future__ import annotations

from typing import Mapping

import torch

from .. import ops
from ..config.model_spec import PartSpec
from .base import Part, PendingNorm, StepContext, add_output, WeightSpec, register_part, release_tensors, require_params

# activation name -> (gated activation of a packed [N, 2 I] row, the same fused with the product)
_ACTIVATIONS = {"silu": (ops.silu_mul, ops.linear_silu_mul)}


class GatedMLP(Part):
    accepts_pending_norm = True
    accumulates_residual = True
    prepares_norm = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "hidden_size", "intermediate_size", "activation")
        self.hidden_size = int(params["hidden_size"])
        self.intermediate_size = int(params["intermediate_size"])
        activation = params["activation"]
        if activation not in _ACTIVATIONS:
            raise ValueError(f"gated_mlp knows the activations {sorted(_ACTIVATIONS)}, not {activation!r}.")
        self._gated_activation, self._gated_product = _ACTIVATIONS[activation]
        self._fused_with_norm = activation == "silu"      # the fused kernel's epilogue is SiLU * up
        self.dtype = dtype
        self.prefix = spec.prefix
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [
            WeightSpec(self.prefix + "gate_proj.weight", (self.intermediate_size, self.hidden_size)),
            WeightSpec(self.prefix + "up_proj.weight", (self.intermediate_size, self.hidden_size)),
            WeightSpec(self.prefix + "down_proj.weight", (self.hidden_size, self.intermediate_size)),
        ]

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Gate rows, then up rows, in one matrix: one product gives ``[N, 2 I]``."""

        names = [self.prefix + "gate_proj.weight", self.prefix + "up_proj.weight"]
        self.w_gate_up = torch.cat([tensors[name] for name in names], dim=0).contiguous()
        self.w_down = tensors[self.prefix + "down_proj.weight"]
        release_tensors(tensors, names)       # the stacked copy serves from here on

    def takes_prepared_norm(self, rows: int) -> bool:
        return self._fused_with_norm and ops.can_use_prepared_norm(rows, self.w_gate_up, gated=True)

    def forward(self, x, ctx: StepContext | None = None, *, residual: torch.Tensor | None = None, norm_after=None):
        """``x``: the normed input, or a ``PendingNorm`` (then the norm becomes a part of the
        gate/up product where one kernel serves the shape: scales prepared by the part
        before, or the product's prologue).  With ``residual`` the output may be added
        into it (the product's epilogue); None is returned then, or, with ``norm_after``
        (the RMSNorm taken of the residual stream next), what that epilogue prepared of it."""

        if isinstance(x, PendingNorm):
            rows = x.shape[0]
            if x.prepared is not None and self.takes_prepared_norm(rows):
                hidden = ops.linear_prepared(x.prepared.weighted, x.prepared.squares, x.norm.eps, self.w_gate_up, gated=True)
            elif x.fusable and self._fused_with_norm and ops.can_fuse_norm(rows, self.w_gate_up, gated=True):
                hidden = ops.linear_normed(x.residual, x.norm.weight, x.norm.eps, self.w_gate_up, gated=True)
            else:
                hidden = self._gated_product(x.materialize(), self.w_gate_up)
        else:
            hidden = self._gated_product(x, self.w_gate_up)
        return add_output(hidden, self.w_down, residual, norm_after)


register_part("feed_forward", "gated_mlp", GatedMLP)
