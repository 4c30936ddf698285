"""Grouped-query attention over the paged cache, with optional per-head norms of
q and k and an optional position encoding (reference: miniserve/model/qwen3.py:56-323).

Order of operations (qwen3.py:174-250): project q, k, v; norm q and k per head;
rotate q and k; write k and v to the cache; attend causally over the cache
(this step's tokens included); project the heads back.
"""

from __future__ import annotations

from typing import Mapping

import torch

from .. import ops
from ..config.model_spec import PartSpec
from .base import (
    HostBatch,
    KVCacheNeed,
    KVCacheView,
    Part,
    PendingNorm,
    StepContext,
    WeightSpec,
    add_output,
    build_part,
    register_part,
    release_tensors,
    require_params,
)
from .norm import RMSNorm
from .rotary import RotaryHalf


class Attention(Part):
    accepts_pending_norm = True
    accumulates_residual = True
    prepares_norm = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype) -> None:
        params = require_params(spec, "hidden_size", "num_heads", "num_kv_heads", "head_dim")
        self.hidden_size = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.num_heads <= 0 or self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ValueError("attention needs num_heads to be a positive multiple of num_kv_heads.")
        scale = params.get("scale")
        self.scale = float(self.head_dim**-0.5 if scale is None else scale)
        window = params.get("window")
        if window is not None and (not isinstance(window, int) or window <= 0):
            raise ValueError("attention window must be a positive integer or None.")
        self.window = window
        page = params.get("block_size")
        if page is not None and (not isinstance(page, int) or page <= 0):
            raise ValueError("attention block_size (tokens a page of its cache holds) must be a positive integer or None.")
        self.block_size = page
        self.dtype = dtype
        self.prefix = spec.prefix
        self.q_norm = build_part("norm", params["q_norm"], dtype) if params.get("q_norm") else None
        self.k_norm = build_part("norm", params["k_norm"], dtype) if params.get("k_norm") else None
        self.position = build_part("position", params["position"], dtype) if params.get("position") else None
        self.w_qkv: torch.Tensor | None = None
        self.w_q: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None
        # The fused kernel covers RMSNorm (or no norm) with one eps and the
        # half-split rotary (or none); anything else is composed from the parts.
        norms = [n for n in (self.q_norm, self.k_norm) if n is not None]
        self._fused = (
            all(isinstance(n, RMSNorm) and n.dim == self.head_dim for n in norms)
            and len({n.eps for n in norms}) <= 1
            and (self.position is None or (isinstance(self.position, RotaryHalf) and self.position.dim == self.head_dim))
            and self.head_dim % 2 == 0
        )

    # -- description ----------------------------------------------------------------
    def sub_parts(self) -> list[Part]:
        return [p for p in (self.q_norm, self.k_norm, self.position) if p is not None]

    def weight_specs(self) -> list[WeightSpec]:
        q_width = self.num_heads * self.head_dim
        kv_width = self.num_kv_heads * self.head_dim
        return [
            WeightSpec(self.prefix + "q_proj.weight", (q_width, self.hidden_size)),
            WeightSpec(self.prefix + "k_proj.weight", (kv_width, self.hidden_size)),
            WeightSpec(self.prefix + "v_proj.weight", (kv_width, self.hidden_size)),
            WeightSpec(self.prefix + "o_proj.weight", (self.hidden_size, q_width)),
        ]

    def cache_need(self) -> KVCacheNeed:
        return KVCacheNeed(self.num_kv_heads, self.head_dim, self.window, self.block_size)

    # The tiled attention kernel walks the runs of tokens of a step in tiles; the tile
    # lists are made on the host once per step, for all attention layers, and travel to
    # the device with the step's other numbers.
    step_tables_key = "attention.tiles"

    @staticmethod
    def step_tables(batch: HostBatch) -> dict[str, list[int]]:
        seqs, tokens, lengths, firsts = ops.query_tiles_host(batch.query_lens, batch.query_start, batch.decode_prefix,
                                                             batch.first_positions)
        return {"attention.tile_seq": seqs, "attention.tile_token": tokens, "attention.tile_length": lengths,
                "attention.tile_first": firsts}

    @staticmethod
    def _tiles(ctx: StepContext):
        if "attention.tiles" not in ctx.scratch:
            seq = ctx.tables.get("attention.tile_seq")
            tiles = None
            if seq is not None and seq.numel() > 0:
                tiles = ops.QueryTiles(seq.numel(), seq, ctx.tables["attention.tile_token"],
                                       ctx.tables["attention.tile_length"], ctx.tables["attention.tile_first"], by_keys=True)
            ctx.scratch["attention.tiles"] = tiles
        return ctx.scratch["attention.tiles"]

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """q, k and v rows are stacked into one matrix, q rows first, then k, then
        v, so one product gives the packed ``[N, (Hq + 2 Hkv) * D]`` row."""

        names = [self.prefix + part + "_proj.weight" for part in ("q", "k", "v")]
        q_rows = tensors[names[0]].shape[0]
        self.w_qkv = torch.cat([tensors[name] for name in names], dim=0).contiguous()
        self.w_q = self.w_qkv[:q_rows]
        self.w_o = tensors[self.prefix + "o_proj.weight"]
        release_tensors(tensors, names)       # the stacked copy serves from here on

    # -- execution ------------------------------------------------------------------
    def takes_prepared_norm(self, rows: int) -> bool:
        return ops.can_use_prepared_norm(rows, self.w_qkv)

    def forward(self, x, ctx: StepContext, cache: KVCacheView, *, residual: torch.Tensor | None = None, norm_after=None):
        """``x``: the normed input ``[N, H]``, or a ``PendingNorm`` (then the norm becomes a
        part of the q/k/v product where one kernel serves the shape: scales prepared by
        the part before, or the product's prologue).  With ``residual`` the output may be
        added into it (the product's epilogue); None is returned then, or, with
        ``norm_after`` (the RMSNorm taken of the residual stream next), what that epilogue
        prepared of it."""

        if not isinstance(cache, KVCacheView):
            raise TypeError("attention needs a paged key/value cache.")
        group = ctx.groups[cache.group]
        n = x.shape[0]
        kv_heads = self.num_kv_heads if cache.write else 0
        w_in = self.w_qkv if cache.write else self.w_q
        if isinstance(x, PendingNorm):
            if x.prepared is not None and ops.can_use_prepared_norm(n, w_in):
                packed = ops.linear_prepared(x.prepared.weighted, x.prepared.squares, x.norm.eps, w_in)
            elif x.fusable and ops.can_fuse_norm(n, w_in):
                packed = ops.linear_normed(x.residual, x.norm.weight, x.norm.eps, w_in)
            else:
                packed = ops.linear(x.materialize(), w_in)
        else:
            packed = ops.linear(x, w_in)
        if self._fused:
            q = ops.qk_norm_rope_append(
                packed,
                num_q_heads=self.num_heads,
                num_kv_heads=kv_heads,
                head_dim=self.head_dim,
                q_weight=None if self.q_norm is None else self.q_norm.weight,
                k_weight=None if self.k_norm is None else self.k_norm.weight,
                eps=next((p.eps for p in (self.q_norm, self.k_norm) if p is not None), 1.0),
                rope=None if self.position is None else self.position.tables(ctx.positions, ctx),
                slot_mapping=group.slot_mapping if cache.write else None,
                key_pool=cache.key if cache.write else None,
                value_pool=cache.value if cache.write else None,
            )
        else:
            q = self._prepare_unfused(packed, ctx, cache, group, kv_heads)
        attended = ops.attention(
            q,
            cache.key,
            cache.value,
            block_table=group.block_table,
            seq_of_token=ctx.seq_of_token,
            positions=ctx.positions,
            scale=self.scale,
            window=self.window,
            decode_prefix=ctx.decode_prefix,
            tiles=self._tiles(ctx),
            max_context=ctx.max_context_len,
        )
        attended = attended.reshape(n, self.num_heads * self.head_dim)
        return add_output(attended, self.w_o, residual, norm_after)

    def _prepare_unfused(self, packed, ctx, cache, group, kv_heads) -> torch.Tensor:
        """Norms and position encoding through their own parts, then the cache write."""

        n = packed.shape[0]
        q_width = self.num_heads * self.head_dim
        kv_width = kv_heads * self.head_dim
        q = packed[:, :q_width].reshape(n, self.num_heads, self.head_dim).contiguous()
        if self.q_norm is not None:
            q = self.q_norm.forward(q)
        if self.position is not None:
            q = self.position.apply(q, ctx.positions)
        if kv_heads == 0:
            return q
        k = packed[:, q_width : q_width + kv_width].reshape(n, kv_heads, self.head_dim).contiguous()
        if self.k_norm is not None:
            k = self.k_norm.forward(k)
        if self.position is not None:
            k = self.position.apply(k, ctx.positions)
        kv = torch.cat([k.reshape(n, kv_width), packed[:, q_width + kv_width :]], dim=1).contiguous()
        ops.qk_norm_rope_append(
            kv,
            num_q_heads=0,
            num_kv_heads=kv_heads,
            head_dim=self.head_dim,
            q_weight=None,
            k_weight=None,
            eps=1.0,
            rope=None,
            slot_mapping=group.slot_mapping,
            key_pool=cache.key,
            value_pool=cache.value,
        )
        return q


register_part("mixer", "attention", Attention)
