"""Interfaces of the parts a layer is built from, and their registries.

A part is constructed from its ``PartSpec`` alone (its sizes and constants), says
which tensors it wants (``weight_specs``), receives them (``load_weights``) and
runs on a flat batch of tokens.  No part knows which model it is in.

Categories and what each must offer:

``norm``              ``forward(x) -> y`` and ``add_forward(residual, delta, *,
                      rows=None, write_back=True) -> y``: the norm of
                      ``residual + delta``; the sum is stored into the 32-bit
                      ``residual`` when ``write_back``.
``position``          ``apply(x [N, heads, dim], positions [N]) -> x'``; no weights.
``mixer``             ``cache_need() -> KVCacheNeed | StateNeed | None`` (or a tuple of
                      needs: pages and a state row, say) and
                      ``forward(x [N, H], ctx: StepContext, cache) -> [N, H]``,
                      ``cache`` being a ``KVCacheView``, a ``StateView``, None, or a
                      tuple of views in the order of the needs.
``feed_forward``      ``forward(x [N, H], ctx) -> [N, H]``.
``block``             the arrangement of one layer's parts around the residual
                      stream: ``forward(residual, delta, ctx, cache) ->
                      (residual, delta)``; the sum ``residual + delta`` is what
                      the next block (or the final norm) starts from.
``embedding``         ``forward(token_ids [N], ctx) -> float32 [N, H]`` (``ctx``: the
                      step's ``StepContext``, for an embedding that adds a term of
                      the position or of another per-token input).
``head``              ``forward(x [R, H]) -> float32 logits [R, V]``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping

import torch

from ..config.model_spec import PartSpec

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")


# ---- what a part says about its tensors ------------------------------------------

@dataclass(frozen=True)
class WeightSpec:
    """One checkpoint tensor that a part wants.

    ``init`` picks the random-weights distribution: the name of a rule
    (``"matrix"`` ~ N(0, 0.02), ``"norm"`` ~ 1 + N(0, 0.1), ``"zeros"``, or one added
    with ``weights.register_init``) or a callable ``(shape, generator, device) ->
    float32 tensor`` of the part's own.  ``keep`` says how the tensor is
    held: ``"compute"`` in the engine's dtype (bfloat16 or float32),
    ``"float32"`` always in 32-bit, ``"int32"`` an integer table.
    ``optional`` tensors may be absent; ``same_as`` names a tensor that an
    optional one must equal bit for bit when it is present (a tied head)."""

    name: str
    shape: tuple[int, ...]
    init: str | Callable[..., torch.Tensor] = "matrix"
    keep: str = "compute"
    optional: bool = False
    same_as: str | None = None


# ---- what a mixer says about its cache -------------------------------------------

PAGE_TOKENS = "tokens"      # in a plane's dims: the number of tokens a page holds


@dataclass(frozen=True)
class PagePlane:
    """One tensor that a mixer keeps per page: ``dims`` is the shape of one page's
    share, with ``PAGE_TOKENS`` where the page's tokens go (``("tokens", 48)``: a vector
    of 48 a token; ``(heads, dim, "tokens")``: tokens innermost)."""

    name: str
    dims: tuple

    def shape(self, block_size: int) -> tuple[int, ...]:
        if sum(1 for dim in self.dims if dim == PAGE_TOKENS) != 1:
            raise ValueError(f"plane {self.name!r}: its dims must name the page's tokens exactly once.")
        return tuple(block_size if dim == PAGE_TOKENS else int(dim) for dim in self.dims)

    def elements_per_token(self) -> int:
        count = 1
        for dim in self.dims:
            count *= 1 if dim == PAGE_TOKENS else int(dim)
        return count


@dataclass(frozen=True)
class KVCacheNeed:
    """What a mixer keeps per token, in pages.  ``window`` None: all tokens are kept; an
    int: only the last ``window`` tokens of a position are ever read, older pages go
    back.  ``block_size``: tokens a page of this mixer's group holds; None = the
    engine's ``kv_block_size`` (a mixer with a short window may want smaller pages).
    ``planes``: the tensors of a page, named by the mixer; None = keys ``[kv_heads,
    tokens, head_dim]`` and values ``[kv_heads, head_dim, tokens]``, what the attention
    kernels of this package read.  A mixer with planes of its own (one latent vector a
    token, keys only) finds them by name in its ``KVCacheView.planes``."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None
    block_size: int | None = None
    planes: tuple[PagePlane, ...] | None = None

    def page_planes(self) -> tuple[PagePlane, ...]:
        if self.planes is not None:
            if not self.planes or len({plane.name for plane in self.planes}) != len(self.planes):
                raise ValueError("a cache need names at least one plane, each once.")
            return self.planes
        return (PagePlane("key", (self.num_kv_heads, PAGE_TOKENS, self.head_dim)),
                PagePlane("value", (self.num_kv_heads, self.head_dim, PAGE_TOKENS)))


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: one tensor of ``shape`` per live request."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVCacheView:
    """One call's slice of its group's pools: keys ``[pages, kv_heads, block_size,
    head_dim]``, values ``[pages, kv_heads, head_dim, block_size]``; for a need with
    planes of its own ``key`` and ``value`` are None and ``planes`` holds each plane's
    ``[pages, *dims]`` under its name (the default planes are there too, as "key" and
    "value")."""

    group: int
    key: torch.Tensor | None
    value: torch.Tensor | None
    block_size: int
    write: bool = True     # False: this call reads another call's cache
    planes: dict[str, torch.Tensor] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if not self.planes:
            self.planes = {name: tensor for name, tensor in (("key", self.key), ("value", self.value)) if tensor is not None}


@dataclass
class StateView:
    """One call's state for every slot: ``[max_num_seqs, *shape]``."""

    tensor: torch.Tensor


# ---- the batch of one step, as parts see it ---------------------------------------

@dataclass
class GroupStepView:
    """Cache metadata of one group for this step."""

    block_table: torch.Tensor    # int32 [S, max_blocks]
    slot_mapping: torch.Tensor   # int32 [N]: page * block_size + offset of each new token


@dataclass(frozen=True)
class HostBatch:
    """What a part may know of a step on the host, before anything is sent: the
    sequences in the order of the batch (those that bring one token first).
    ``recorded``: the batch stands for every replay of a recorded step of single
    tokens; then the positions are not known (``first_positions`` is None) and the
    tables made from it are made once."""

    query_lens: tuple[int, ...]         # tokens that each sequence brings
    query_start: tuple[int, ...]        # index of each sequence's first token in the batch, and the total
    first_positions: tuple[int, ...] | None    # absolute position of each sequence's first token
    decode_prefix: int                  # sequences at the front that bring exactly one token
    recorded: bool = False


@dataclass
class StepContext:
    """A flat ragged batch: ``N`` tokens of ``S`` sequences, each sequence's tokens
    contiguous and at consecutive absolute positions.  Sequences that bring one
    token come first (``decode_prefix`` of them), so that kernels made for single
    tokens and kernels made for runs of tokens can each take their share.

    The host copies exist for launch decisions.  In a *recorded* step (``recorded``:
    a graph that is replayed for many steps of single tokens) only what holds for
    every replay is given: ``query_lens`` and ``query_start_host`` (one token each);
    the other host copies are None, and ``max_context_len`` is the bound that no
    request exceeds.  A part that needs per-request values there reads the device
    tensors (``state_slots``, ``positions``, ``context_lens``)."""

    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor       # int32 [N]
    positions: torch.Tensor       # int32 [N], absolute
    seq_of_token: torch.Tensor    # int32 [N]
    query_start: torch.Tensor     # int32 [S + 1]
    context_lens: torch.Tensor    # int32 [S], length after this step
    state_slots: torch.Tensor     # int32 [S]
    groups: list[GroupStepView]
    # host copies, for launch decisions
    query_lens: list[int] = field(default_factory=list)
    context_lens_host: list[int] | None = field(default_factory=list)
    query_start_host: list[int] = field(default_factory=list)
    state_slots_host: list[int] | None = field(default_factory=list)
    first_positions_host: list[int] | None = field(default_factory=list)
    decode_prefix: int = 0
    recorded: bool = False
    context_bound: int | None = None      # recorded steps: the longest context any replay can have
    # integer tables that parts asked for (``step_tables``), sent with the step's other numbers
    tables: dict[str, torch.Tensor] = field(default_factory=dict)
    # what parts compute once per step and share between layers (position tables)
    scratch: dict = field(default_factory=dict)

    @property
    def max_query_len(self) -> int:
        return max(self.query_lens)

    @property
    def max_context_len(self) -> int:
        if self.context_lens_host is None:
            if self.context_bound is None:
                raise RuntimeError("a recorded step has no per-request context lengths on the host.")
            return self.context_bound
        return max(self.context_lens_host)


# ---- a norm that is not yet taken ------------------------------------------------------

class PreparedNorm:
    """What a part that added its output into the residual stream left for the RMSNorm
    behind it (``ops.linear_norm_ahead``): ``weighted`` = the norm's weight times the new
    residual values, rounded to the model's dtype, and ``squares``, partial sums of their
    squares.  ``ops.linear_prepared`` makes a product of the norm from the two; the norm
    itself can always still be taken from the residual stream."""

    def __init__(self, norm, weighted: torch.Tensor, squares: torch.Tensor) -> None:
        self.norm = norm
        self.weighted = weighted
        self.squares = squares


class PendingNorm:
    """``norm(residual + delta)``, not yet computed.  A block hands it to a mixer or a
    feed-forward that sets ``accepts_pending_norm = True``; such a part may fuse the
    norm into its first product (when ``fusable``: an RMSNorm whose input is the bare
    residual stream; ``prepared``: what the part before left for exactly this norm, or
    None) or call :meth:`materialize` for the normed tensor.  Every other part receives
    the materialised tensor."""

    def __init__(self, norm, residual: torch.Tensor, delta: "torch.Tensor | PreparedNorm | None") -> None:
        self.norm = norm
        self.residual = residual
        self.prepared: PreparedNorm | None = None
        if isinstance(delta, PreparedNorm):
            # made for another norm than this one: the residual stream holds the sum all the same
            self.prepared = delta if delta.norm is norm else None
            delta = None
        self.delta = delta
        self._value: torch.Tensor | None = None

    @property
    def fusable(self) -> bool:
        return self.delta is None and hasattr(self.norm, "eps") and getattr(self.norm, "weight", None) is not None

    @property
    def shape(self):
        return self.residual.shape

    def materialize(self) -> torch.Tensor:
        if self._value is None:
            self._value = self.norm.add_forward(self.residual, self.delta)
            self.delta = None       # the sum has been stored into the residual stream
        return self._value


def add_output(hidden: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor | None, norm_after=None):
    """The last product of a mixer or feed-forward, ``hidden @ weight^T``.  Without
    ``residual`` it is returned.  With it, the product is added into the residual stream
    by its own epilogue where a kernel does that, and None is returned, or, when
    ``norm_after`` is an RMSNorm with a weight and the kernel serves the shape, the
    ``PreparedNorm`` that the same epilogue made for it."""

    from .. import ops

    rows = hidden.shape[0]
    if residual is None or not ops.can_accumulate(rows, weight):
        return ops.linear(hidden, weight)
    norm_weight = getattr(norm_after, "weight", None)
    if norm_weight is not None and hasattr(norm_after, "eps") and ops.can_prepare_norm(rows, weight):
        return PreparedNorm(norm_after, *ops.linear_norm_ahead(hidden, weight, residual, norm_weight))
    ops.linear(hidden, weight, accumulate_into=residual)
    return None


# ---- registries -------------------------------------------------------------------

_REGISTRIES: dict[str, dict[str, Callable[..., Any]]] = {category: {} for category in CATEGORIES}


def register_part(category: str, kind: str, factory: Callable[..., Any]) -> None:
    """Register ``factory(spec: PartSpec, dtype: torch.dtype) -> part`` under ``kind``."""

    if category not in _REGISTRIES:
        raise ValueError(f"unknown part category {category!r}; one of {CATEGORIES}.")
    _REGISTRIES[category][kind] = factory


def unregister_part(category: str, kind: str) -> None:
    _REGISTRIES[category].pop(kind, None)


def build_part(category: str, spec: PartSpec, dtype: torch.dtype) -> Any:
    try:
        factory = _REGISTRIES[category][spec.kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES.get(category, {}))) or "none"
        raise KeyError(f"no {category} part of kind {spec.kind!r} is registered (known: {known}).") from None
    return factory(spec, dtype)


def registered_parts(category: str) -> tuple[str, ...]:
    return tuple(sorted(_REGISTRIES[category]))


def require_params(spec: PartSpec, *names: str) -> Mapping[str, Any]:
    missing = [name for name in names if name not in spec.params]
    if missing:
        raise ValueError(f"part {spec.kind!r} lacks parameters {missing}.")
    return spec.params


def release_tensors(tensors, names) -> None:
    """A part that has copied checkpoint tensors into a layout of its own (stacked
    matrices) drops the originals from the mapping it was given, where the mapping
    lets it: their memory is free before the cache pool is sized."""

    if hasattr(tensors, "pop"):
        for name in names:
            tensors.pop(name, None)


class Part:
    """Base of all parts: no weights, nothing to load."""

    def weight_specs(self) -> list[WeightSpec]:
        return []

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        return None

    def sub_parts(self) -> list["Part"]:
        return []


def collect_weight_specs(part: Part) -> list[WeightSpec]:
    specs = list(part.weight_specs())
    for child in part.sub_parts():
        specs.extend(collect_weight_specs(child))
    return specs


def load_part_weights(part: Part, tensors: Mapping[str, torch.Tensor]) -> None:
    part.load_weights(tensors)
    for child in part.sub_parts():
        load_part_weights(child, tensors)


def build_block(layer, dtype: torch.dtype) -> Any:
    """A block factory takes the whole ``LayerSpec`` (``layer.block`` is its kind)."""

    try:
        factory = _REGISTRIES["block"][layer.block]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES["block"])) or "none"
        raise KeyError(f"no block arrangement {layer.block!r} is registered (known: {known}).") from None
    return factory(layer, dtype)
