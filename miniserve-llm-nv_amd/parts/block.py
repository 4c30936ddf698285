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
    product) and then returns None instead of the output.  Such a part that also sets
    ``prepares_norm`` is told the norm that will be taken of ``h`` next (``norm_after``,
    when the part behind that norm says by ``takes_prepared_norm(rows)`` that it has a use
    for it) and may return a ``PreparedNorm`` for it instead of None.  The norm after the
    block's last part belongs to whoever runs the block next: the model passes it in as
    ``norm_after`` when the next block sets ``first_norm`` and ``takes_prepared_norm``."""

    accepts_norm_after = True

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

    @property
    def first_norm(self):
        return self.pre_mixer

    def takes_prepared_norm(self, rows: int) -> bool:
        """Whether the block's first part has a use for a ``PreparedNorm`` of ``first_norm``."""

        return self._takes(self.mixer, rows)

    @staticmethod
    def _takes(part, rows: int) -> bool:
        asked = getattr(part, "takes_prepared_norm", None)
        return bool(getattr(part, "accepts_pending_norm", False) and asked is not None and asked(rows))

    @staticmethod
    def _input(part, norm, residual, delta):
        pending = PendingNorm(norm, residual, delta)
        return pending if getattr(part, "accepts_pending_norm", False) else pending.materialize()

    @staticmethod
    def _run(part, x, extra, residual, norm_after):
        if not getattr(part, "accumulates_residual", False):
            return part.forward(x, *extra)
        if norm_after is not None and getattr(part, "prepares_norm", False):
            return part.forward(x, *extra, residual=residual, norm_after=norm_after)
        return part.forward(x, *extra, residual=residual)

    def forward(self, residual: torch.Tensor, delta, ctx: StepContext, cache, *, norm_after=None):
        rows = residual.shape[0]
        x = self._input(self.mixer, self.pre_mixer, residual, delta)
        between = self.pre_feed_forward if self._takes(self.feed_forward, rows) else None
        mixed = self._run(self.mixer, x, (ctx, cache), residual, between)
        x = self._input(self.feed_forward, self.pre_feed_forward, residual, mixed)
        return residual, self._run(self.feed_forward, x, (ctx,), residual, norm_after)


register_part("block", "prenorm", PreNormBlock)
