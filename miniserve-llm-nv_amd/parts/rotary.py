"""Half-split ("NeoX") rotary position embedding from absolute positions
(reference: miniserve/model/rope.py:8-52)."""

from __future__ import annotations

import torch

from .. import ops
from ..config.model_spec import PartSpec
from .base import Part, register_part, require_params


def inverse_frequencies(dim: int, theta: float) -> torch.Tensor:
    """``inv_freq[i] = 1 / theta^(2i/dim)`` in float32, computed exactly as the
    reference does (rope.py:24-25) so that angles agree to the bit."""

    exponents = torch.arange(0, dim, 2, dtype=torch.float32) / dim
    return 1.0 / (theta**exponents)


class RotaryHalf(Part):
    """Pairs ``(i, i + dim/2)`` are rotated by ``position * inv_freq[i]``."""

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "dim", "theta")
        self.dim = int(params["dim"])
        self.theta = float(params["theta"])
        if self.dim <= 0 or self.dim % 2 or not self.theta > 0:
            raise ValueError("rotary needs an even dim > 0 and theta > 0.")
        self.dtype = dtype
        self._inv_freq_host = inverse_frequencies(self.dim, self.theta)
        self._inv_freq: torch.Tensor | None = None

    def inv_freq(self, device: torch.device) -> torch.Tensor:
        if self._inv_freq is None or self._inv_freq.device != device:
            self._inv_freq = self._inv_freq_host.to(device)
        return self._inv_freq

    def tables(self, positions: torch.Tensor, ctx=None) -> tuple[torch.Tensor, torch.Tensor]:
        """cos and sin ``[N, dim/2]`` (float32) for ``positions``; with a step context
        they are made once and shared by every layer of the step."""

        if ctx is None:
            return ops.rope_table(positions, self.inv_freq(positions.device))
        key = ("rotary_half", self.dim, self.theta)
        if key not in ctx.scratch:
            ctx.scratch[key] = ops.rope_table(ctx.positions, self.inv_freq(ctx.positions.device))
        return ctx.scratch[key]

    def apply(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """``x [N, heads, dim]`` rotated by ``positions [N]`` (int32)."""

        n, heads, dim = x.shape
        if dim != self.dim:
            raise ValueError(f"rotary of dim {self.dim} applied to head size {dim}.")
        return ops.qk_norm_rope_append(
            x.reshape(n, heads * dim),
            num_q_heads=heads,
            num_kv_heads=0,
            head_dim=dim,
            q_weight=None,
            k_weight=None,
            eps=1.0,
            rope=self.tables(positions),
        )


register_part("position", "rotary_half", RotaryHalf)
