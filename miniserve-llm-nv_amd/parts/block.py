"""Arrangements of one layer's parts around the residual stream."""

from __future__ import annotations

import torch

from ..config.model_spec import LayerSpec
from .base import Part, StepContext, build_part, register_part


class PreNormBlock(Part):
    """``h <- h + mixer(norm(h)); h <- h + feed_forward(norm(h))``
    (reference: miniserve/model/qwen3.py:342-347).

    The residual stream ``h`` is float32.  A block receives ``(h, delta)`` with
    ``delta`` the previous block's last output, not yet added; the add is fused
    into the next norm, and the block hands its own last output on the same way."""

    def __init__(self, layer: LayerSpec, dtype: torch.dtype) -> None:
        for role in ("pre_mixer", "pre_feed_forward"):
            if role not in layer.norms:
                raise ValueError(f"a prenorm block needs the norm {role!r}.")
        self.pre_mixer = build_part("norm", layer.norms["pre_mixer"], dtype)
        self.mixer = build_part("mixer", layer.mixer, dtype)
        self.pre_feed_forward = build_part("norm", layer.norms["pre_feed_forward"], dtype)
        self.feed_forward = build_part("feed_forward", layer.feed_forward, dtype)

    def sub_parts(self) -> list[Part]:
        return [self.pre_mixer, self.mixer, self.pre_feed_forward, self.feed_forward]

    def forward(self, residual: torch.Tensor, delta: torch.Tensor | None, ctx: StepContext, cache):
        x = self.pre_mixer.add_forward(residual, delta)
        mixed = self.mixer.forward(x, ctx, cache)
        x = self.pre_feed_forward.add_forward(residual, mixed)
        return residual, self.feed_forward.forward(x, ctx)


register_part("block", "prenorm", PreNormBlock)
