"""Arrangements of one layer's parts around the residual stream."""

from __future__ import annotations

import torch

from ..config.model_spec import LayerSpec
from .base import Part, PendingNorm, StepContext, build_part, register_part


class PreNormBlock(Part):
    """``h <- h + mixer(norm(h)); h <- h + feed_forward(norm(h))``
    (reference: miniserve/model/qwen3.py:342-347).

    The residual stream ``h`` is float32.  A block receives ``(h, delta)`` with
    ``delta`` the previous block's last output, not yet added (or None when it has
    been added); the add is fused into the next norm, and the block hands its own
    last output on the same way.

    Two fusions are offered to parts that ask for them by attribute.
    ``accepts_pending_norm``: the part gets the norm as a ``PendingNorm`` and may make
    it the prologue of its first product.  ``accumulates_residual``: the part gets
    ``residual=h``, may add its output into ``h`` itself (the epilogue of its last
    product) and then returns None instead of the output."""

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

    @staticmethod
    def _input(part, norm, residual, delta):
        pending = PendingNorm(norm, residual, delta)
        return pending if getattr(part, "accepts_pending_norm", False) else pending.materialize()

    def forward(self, residual: torch.Tensor, delta: torch.Tensor | None, ctx: StepContext, cache):
        x = self._input(self.mixer, self.pre_mixer, residual, delta)
        if getattr(self.mixer, "accumulates_residual", False):
            mixed = self.mixer.forward(x, ctx, cache, residual=residual)
        else:
            mixed = self.mixer.forward(x, ctx, cache)
        x = self._input(self.feed_forward, self.pre_feed_forward, residual, mixed)
        if getattr(self.feed_forward, "accumulates_residual", False):
            return residual, self.feed_forward.forward(x, ctx, residual=residual)
        return residual, self.feed_forward.forward(x, ctx)


register_part("block", "prenorm", PreNormBlock)
