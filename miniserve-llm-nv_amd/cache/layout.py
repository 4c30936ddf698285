"""What the model's calls need of the cache, sorted into groups.

A *group* is a set of calls with the same need (the planes of a page, window, page
size): they share one page pool, one allocator and one block table per request.
Calls with a fixed-size state own no pages; they get a tensor with one row per state
slot.  A call that reads another call's cache owns nothing.  A call may need several
things at once (pages and a state row): it gets a tuple of views, one per need.
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
    """Where call ``call`` finds its cache: ``kind`` is "kv", "state", "none", or "many"
    (then ``parts`` holds a placement for each of the call's needs, in their order)."""

    call: int
    kind: str
    group: int = -1          # kv: the group
    index: int = -1          # kv: position inside the group's pool; state: index of the state tensor
    write: bool = True       # kv: False when the call reads another call's cache
    parts: tuple = ()


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

        def place(call: int, need, cache_from) -> CallPlacement:
            if need is None:
                return CallPlacement(call, "none")
            if isinstance(need, StateNeed):
                states.append(need)
                return CallPlacement(call, "state", index=len(states) - 1)
            if isinstance(need, KVCacheNeed):
                if cache_from is not None:
                    source = placements[cache_from]
                    if source.kind != "kv" or not source.write:
                        raise ValueError(f"call {call} reads the cache of call {cache_from}, which owns none.")
                    return CallPlacement(call, "kv", source.group, source.index, write=False)
                need.page_planes()      # a need with wrong planes is refused here, before anything is allocated
                group = by_need.get(need)
                if group is None:
                    group = KVGroup(len(groups), need)
                    groups.append(group)
                    by_need[need] = group
                group.calls.append(call)
                return CallPlacement(call, "kv", group.index, len(group.calls) - 1)
            raise TypeError(f"call {call}: unknown cache need {need!r}.")

        for item in needs:
            if isinstance(item.need, (tuple, list)):
                if item.cache_from is not None:
                    raise ValueError(f"call {item.call} has several needs and cannot read another call's cache.")
                parts = tuple(place(item.call, need, None) for need in item.need)
                placements.append(CallPlacement(item.call, "many", parts=parts))
            else:
                placements.append(place(item.call, item.need, item.cache_from))
        return cls(groups, states, placements)

    def bytes_per_token(self, itemsize: int) -> int:
        """Bytes that one token takes in the pages of all groups: keys and values with
        the default planes (reference: miniserve/kv/layout.py:59-60)."""

        return sum(
            len(g.calls) * sum(plane.elements_per_token() for plane in g.need.page_planes()) * itemsize
            for g in self.groups
        )
