"""What the model's calls need of the cache, sorted into groups.

A *group* is a set of calls with the same need (kv heads, head size, window):
they share one page pool, one allocator and one block table per request.  Calls
with a fixed-size state own no pages; they get a tensor with one row per state
slot.  A call that reads another call's cache owns nothing.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

from ..parts.base import KVCacheNeed, StateNeed


@dataclass
class KVGroup:
    index: int
    need: KVCacheNeed
    calls: list[int] = field(default_factory=list)     # calls that own a cache, in run order

    @property
    def window(self) -> int | None:
        return self.need.window


@dataclass(frozen=True)
class CallPlacement:
    """Where call ``call`` finds its cache: ``kind`` is "kv", "state" or "none"."""

    call: int
    kind: str
    group: int = -1          # kv: the group
    index: int = -1          # kv: position inside the group's pool; state: index of the state tensor
    write: bool = True       # kv: False when the call reads another call's cache


@dataclass
class CacheLayout:
    groups: list[KVGroup]
    states: list[StateNeed]
    placements: list[CallPlacement]

    @classmethod
    def from_needs(cls, needs: Sequence) -> "CacheLayout":
        """``needs``: objects with ``call``, ``need`` and ``cache_from`` (the model's
        ``cache_needs()``), in run order."""

        groups: list[KVGroup] = []
        by_need: dict[KVCacheNeed, KVGroup] = {}
        states: list[StateNeed] = []
        placements: list[CallPlacement] = []
        for item in needs:
            need = item.need
            if need is None:
                placements.append(CallPlacement(item.call, "none"))
            elif isinstance(need, StateNeed):
                states.append(need)
                placements.append(CallPlacement(item.call, "state", index=len(states) - 1))
            elif isinstance(need, KVCacheNeed):
                if item.cache_from is not None:
                    source = placements[item.cache_from]
                    if source.kind != "kv" or not source.write:
                        raise ValueError(f"call {item.call} reads the cache of call {item.cache_from}, which owns none.")
                    placements.append(CallPlacement(item.call, "kv", source.group, source.index, write=False))
                    continue
                group = by_need.get(need)
                if group is None:
                    group = KVGroup(len(groups), need)
                    groups.append(group)
                    by_need[need] = group
                group.calls.append(item.call)
                placements.append(CallPlacement(item.call, "kv", group.index, len(group.calls) - 1))
            else:
                raise TypeError(f"call {item.call}: unknown cache need {need!r}.")
        return cls(groups, states, placements)

    def bytes_per_token(self, itemsize: int) -> int:
        """Bytes of keys and values that one token takes over all groups
        (reference: miniserve/kv/layout.py:59-60)."""

        return sum(2 * len(g.calls) * g.need.num_kv_heads * g.need.head_dim * itemsize for g in self.groups)
