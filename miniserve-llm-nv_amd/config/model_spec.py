"""Architecture-independent description of a decoder, as plain data.

A configuration class turns its ``config.json`` into a :class:`ModelSpec`; the
model assembler reads nothing else.  Every size and constant of a part travels
in its :class:`PartSpec`, so a part never learns which model it is in, and two
layers of one model may name different mixers or feed-forwards.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Any, Mapping


def _freeze(params: Mapping[str, Any]) -> Mapping[str, Any]:
    return MappingProxyType(dict(params))


@dataclass(frozen=True)
class PartSpec:
    """One part: its kind (a name in the registry of its category), its sizes and
    constants, and the checkpoint-name prefix of its tensors."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""

    def __post_init__(self) -> None:
        if not isinstance(self.kind, str) or not self.kind:
            raise ValueError("PartSpec.kind must be a non-empty string.")
        object.__setattr__(self, "params", _freeze(self.params))


@dataclass(frozen=True)
class LayerSpec:
    """One layer with weights of its own: how its parts are arranged (``block``),
    its mixer, its feed-forward and its norms by role."""

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]

    def __post_init__(self) -> None:
        object.__setattr__(self, "norms", _freeze(self.norms))


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` and may
    repeat.  ``cache_from`` names an EARLIER entry of the order whose cache this
    call reads instead of keeping one of its own; ``None`` = own cache."""

    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    order: tuple[LayerCall, ...]
    final_norm: PartSpec
    head: PartSpec

    def __post_init__(self) -> None:
        if not self.layers or not self.order:
            raise ValueError("A model needs at least one layer and one call.")
        for index, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"order[{index}] names layer {call.layer}, which does not exist.")
            if call.cache_from is not None:
                if not 0 <= call.cache_from < index:
                    raise ValueError(f"order[{index}].cache_from must name an earlier call.")
                if self.order[call.cache_from].cache_from is not None:
                    raise ValueError(f"order[{index}].cache_from must name a call that owns its cache.")
