"""A decoder assembled from a ``ModelSpec``: embedding, the layers in their run
order, final norm and head.  Which architecture the spec came from is unknown
here (reference for the Qwen3 arrangement: miniserve/model/qwen3.py:409-613)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, Sequence

import torch

from ..config.model_spec import ModelSpec
from .base import (
    KVCacheNeed,
    Part,
    PreparedNorm,
    StateNeed,
    StepContext,
    WeightSpec,
    build_block,
    build_part,
    collect_weight_specs,
    load_part_weights,
)

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass(frozen=True)
class CallCacheNeed:
    """What entry ``call`` of the run order needs of the cache manager."""

    call: int
    need: KVCacheNeed | StateNeed | None | tuple     # a tuple: several needs at once (pages and a state row)
    cache_from: int | None


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: str | torch.dtype) -> None:
        self.spec = spec
        self.dtype = TORCH_DTYPES[dtype] if isinstance(dtype, str) else dtype
        if self.dtype not in TORCH_DTYPES.values():
            raise ValueError("the model runs in bfloat16 or float32.")
        self.embedding = build_part("embedding", spec.embedding, self.dtype)
        self.layers = [build_block(layer, self.dtype) for layer in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, self.dtype)
        self.head = build_part("head", spec.head, self.dtype)
        self.order = spec.order
        self.device: torch.device | None = None

    # -- description ----------------------------------------------------------------
    def parts(self) -> list[Part]:
        return [self.embedding, *self.layers, self.final_norm, self.head]

    def weight_specs(self) -> list[WeightSpec]:
        """Every tensor the model wants, in a fixed order (embedding, layers, final
        norm, head); a name that two parts share is listed once."""

        seen: dict[str, WeightSpec] = {}
        for part in self.parts():
            for spec in collect_weight_specs(part):
                known = seen.get(spec.name)
                if known is None:
                    seen[spec.name] = spec
                elif known.shape != spec.shape:
                    raise ValueError(f"tensor {spec.name} is wanted with shapes {known.shape} and {spec.shape}.")
        return list(seen.values())

    def cache_needs(self) -> list[CallCacheNeed]:
        needs = []
        for index, call in enumerate(self.order):
            mixer = self.layers[call.layer].mixer
            need = mixer.cache_need() if hasattr(mixer, "cache_need") else None
            if call.cache_from is not None:
                source = self.layers[self.order[call.cache_from].layer].mixer
                if source.cache_need() != need or not isinstance(need, KVCacheNeed):
                    raise ValueError(f"call {index} cannot read the cache of call {call.cache_from}: needs differ.")
            needs.append(CallCacheNeed(index, need, call.cache_from))
        return needs

    def step_tables(self, batch) -> dict[str, list[int]]:
        """Integer tables that parts want made on the host for this step (a
        ``HostBatch``) and sent with its other numbers; they find them in
        ``ctx.tables`` under the names they gave.  A mixer or feed-forward offers
        ``step_tables(batch) -> {name: integers}`` and ``step_tables_key`` (parts with
        the same key want the same tables: they are made once)."""

        tables: dict[str, list[int]] = {}
        seen: set = set()
        for layer in self.layers:
            for part in (getattr(layer, "mixer", None), getattr(layer, "feed_forward", None)):
                provider = getattr(part, "step_tables", None)
                if provider is None:
                    continue
                key = getattr(part, "step_tables_key", id(part))
                if key in seen:
                    continue
                seen.add(key)
                for name, values in provider(batch).items():
                    if name in tables:
                        raise ValueError(f"two parts name a step table {name!r}.")
                    tables[name] = values
        return tables

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            load_part_weights(part, tensors)
        self.device = next(iter(tensors.values())).device

    # -- execution ------------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: Sequence, logit_rows: torch.Tensor | None) -> torch.Tensor | None:
        """Runs the ``N`` tokens of ``ctx`` through every call of the order;
        ``caches[i]`` is the cache of call ``i``.  Returns float32 logits
        ``[R, V]`` for the rows ``logit_rows`` (int32 indices into the ``N``
        tokens), or None when no row is wanted; the final norm and the head run
        on those rows alone."""

        residual = self.embedding.forward(ctx.token_ids, ctx)
        delta = None
        rows = residual.shape[0]
        for index, call in enumerate(self.order):
            block = self.layers[call.layer]
            # the norm that the next block takes first: this block's last part may prepare it
            norm_after = None
            if index + 1 < len(self.order) and getattr(block, "accepts_norm_after", False):
                following = self.layers[self.order[index + 1].layer]
                takes = getattr(following, "takes_prepared_norm", None)
                if takes is not None and takes(rows):
                    norm_after = getattr(following, "first_norm", None)
            if norm_after is not None:
                residual, delta = block.forward(residual, delta, ctx, caches[index], norm_after=norm_after)
            else:
                residual, delta = block.forward(residual, delta, ctx, caches[index])
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        if isinstance(delta, PreparedNorm):
            delta = None            # the residual stream holds the sum
        normed = self.final_norm.add_forward(residual, delta, rows=logit_rows, write_back=False)
        return self.head.forward(normed)
