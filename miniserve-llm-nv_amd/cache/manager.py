"""The cache manager: pages for keys and values, a block table per request and
group, and numbered slots for per-request state of fixed size.

A step is a transaction, as in the reference (miniserve/kv/manager.py:119-192,
kv/paged.py:59-104): ``prepare_step`` reserves the missing pages tentatively,
computes the slot of every new token and keeps a copy of the requests' state rows,
``commit_step`` makes the pages part of the tables and advances the committed
lengths, ``abort_step`` gives exactly the step's new pages back and restores the
state.  Beyond the reference: groups of calls with different
needs have pools, allocators and tables of their own; a group with a window gives
pages back as soon as no later position can read them; every live request holds a
numbered state slot.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping, Sequence

from ..parts.base import KVCacheView, StateView
from .allocator import OutOfPagesError, PageAllocator
from .layout import CacheLayout
from .table import BlockTable


class CacheError(RuntimeError):
    pass


@dataclass(frozen=True)
class CapacitySnapshot:
    """What the scheduler may know: numbers only (reference: miniserve/kv/base.py:14-36).
    Everything is per cache group; a group has its own page size."""

    block_sizes: tuple[int, ...]       # tokens a page holds
    total_blocks: tuple[int, ...]
    free_blocks: tuple[int, ...]
    free_slots: int
    total_slots: int
    held_blocks: Mapping[str, tuple[int, ...]] = field(default_factory=dict)   # per live request
    windows: tuple[int | None, ...] = ()   # the window of the group's layers, None = all keys are kept

    def most_pages_held(self, total_tokens: int, step_tokens: int) -> tuple[int, ...]:
        """The most pages of each group that one request of ``total_tokens`` holds at any
        time when no step brings more than ``step_tokens``: all its pages where all keys
        are kept; where a window has passed, only the pages from the oldest key that the
        step's first token still sees to the step's last token (an edge page more, since
        that span may begin anywhere inside a page)."""

        windows = self.windows or (None,) * len(self.total_blocks)
        held = []
        for block_size, window in zip(self.block_sizes, windows):
            whole = -(-total_tokens // block_size)
            if window is None:
                held.append(whole)
            else:
                span = min(total_tokens, window - 1 + min(step_tokens, total_tokens))
                held.append(min(whole, -(-span // block_size) + 1))
        return tuple(held)

    def pages_for(self, before: int, after: int) -> tuple[int, ...]:
        """New pages of each group that growing a request from ``before`` to ``after`` tokens takes."""

        return tuple(-(-after // size) - -(-before // size) for size in self.block_sizes)

    def room_for(self, before: int, free_pages: Sequence[int]) -> int:
        """Tokens that a request of ``before`` tokens can grow by with ``free_pages``
        new pages per group: the rest of its last page and the free pages, in the
        group where that is least."""

        return min(
            ((-before) % size + max(free, 0) * size for size, free in zip(self.block_sizes, free_pages)),
            default=1 << 60,
        )

    @property
    def min_free_blocks(self) -> int:
        return min(self.free_blocks) if self.free_blocks else 1 << 60


@dataclass(frozen=True)
class StepItem:
    request_id: str
    start: int        # first new position = tokens already committed
    end: int          # length after the step


@dataclass
class SequenceStepMeta:
    """One request's share of a prepared step."""

    request_id: str
    state_slot: int
    before: int
    after: int
    block_tables: list[tuple[int, ...]]     # per group, committed + tentative pages
    slot_mappings: list[tuple[int, ...]]    # per group, one slot per new token
    new_pages: list[list[int]]              # per group


@dataclass
class StepReservation:
    step_id: int
    sequences: list[SequenceStepMeta] = field(default_factory=list)
    closed: bool = False
    # per state tensor: (slot indices on the device, the rows as they were before the step)
    state_before: list = field(default_factory=list)


@dataclass
class _Live:
    request_id: str
    state_slot: int
    committed: int = 0
    tables: list[BlockTable] = field(default_factory=list)
    pending: bool = False


class CacheManager:
    def __init__(
        self,
        layout: CacheLayout,
        *,
        block_size: int,
        num_blocks: int | Sequence[int],
        max_num_seqs: int,
        max_model_len: int,
    ) -> None:
        if block_size <= 0 or max_num_seqs <= 0 or max_model_len <= 0:
            raise ValueError("block_size, max_num_seqs and max_model_len must be positive.")
        self.layout = layout
        self.block_size = block_size          # the engine's page size; a group's need may name its own
        self.block_sizes = tuple(
            block_size if group.need.block_size is None else group.need.block_size for group in layout.groups
        )
        if any(type(size) is not int or size <= 0 for size in self.block_sizes):
            raise ValueError(f"page sizes must be positive whole numbers, not {self.block_sizes}.")
        if isinstance(num_blocks, int):
            # one number: pages of the engine's size; a group with pages of its own size gets as many tokens
            counts = [max(1, num_blocks * block_size // size) for size in self.block_sizes]
        else:
            counts = list(num_blocks)
        if len(counts) != len(layout.groups):
            raise ValueError("num_blocks must give one count per cache group.")
        self.num_blocks = tuple(counts)
        self.max_num_seqs = max_num_seqs
        self.max_model_len = max_model_len
        self.allocators = [PageAllocator(count) for count in counts]
        self._free_slots = list(range(max_num_seqs - 1, -1, -1))   # pop() gives the lowest
        self._live: dict[str, _Live] = {}
        self._next_step_id = 0
        self._open: StepReservation | None = None
        # storage, attached by allocate_storage()
        self.pools: list[dict] = []        # per group: plane name -> [calls, pages + 1, *plane shape]
        self.key_pools: list = []          # the "key" and "value" planes of the groups that have them
        self.value_pools: list = []
        self.state_tensors: list = []

    # ---- storage --------------------------------------------------------------------
    def allocate_storage(self, dtype, device) -> None:
        """Per group one pool for every plane that the group's need names,
        ``[calls, pages + 1, *plane shape]``; with the default planes a key pool
        ``[calls, pages + 1, kv_heads, block_size, head_dim]`` and a value pool
        ``[calls, pages + 1, kv_heads, head_dim, block_size]`` (values lie
        transposed inside a page: the matrix-core kernels read 4 consecutive keys
        of one column in one load).  Allocated once and never initialised (a page's content is read only below the
        committed length; reference: miniserve/kv/paged.py:39-41), and zeroed
        state tensors ``[slots + 1, *shape]``.  The last page of a pool and the last
        state slot are spare: no request ever holds them, and rows that only fill a
        recorded step up to its size write there (:meth:`spare_page`,
        :attr:`spare_state_slot`)."""

        import torch

        self.pools, self.key_pools, self.value_pools, self.state_tensors = [], [], [], []
        for group, count, page in zip(self.layout.groups, self.num_blocks, self.block_sizes):
            made = {
                plane.name: torch.empty((len(group.calls), count + 1, *plane.shape(page)), dtype=dtype, device=device)
                for plane in group.need.page_planes()
            }
            self.pools.append(made)
            if "key" in made:
                self.key_pools.append(made["key"])
            if "value" in made:
                self.value_pools.append(made["value"])
        for need in self.layout.states:
            self.state_tensors.append(torch.zeros((self.max_num_seqs + 1, *need.shape), dtype=need.dtype, device=device))

    def page_pools(self) -> list:
        """Every page pool of every group (tests poison them before a run)."""

        return [pool for made in self.pools for pool in made.values()]

    def spare_page(self, group: int) -> int:
        """The page of ``group``'s pools that belongs to no request."""

        return self.num_blocks[group]

    @property
    def spare_state_slot(self) -> int:
        """The state slot that belongs to no request."""

        return self.max_num_seqs

    def call_views(self) -> list:
        """The cache of every call of the run order: ``KVCacheView``, ``StateView``, None,
        or a tuple of them for a call with several needs."""

        def view(placement):
            if placement.kind == "kv":
                planes = {name: pool[placement.index] for name, pool in self.pools[placement.group].items()}
                return KVCacheView(
                    group=placement.group,
                    key=planes.get("key"),
                    value=planes.get("value"),
                    block_size=self.block_sizes[placement.group],
                    write=placement.write,
                    planes=planes,
                )
            if placement.kind == "state":
                return StateView(self.state_tensors[placement.index])
            if placement.kind == "many":
                return tuple(view(part) for part in placement.parts)
            return None

        return [view(placement) for placement in self.layout.placements]

    # ---- admission and release --------------------------------------------------------
    def admit(self, request_id: str) -> int:
        """Give ``request_id`` a state slot and empty tables; returns the slot."""

        if request_id in self._live:
            raise CacheError(f"request {request_id!r} is already live.")
        if not self._free_slots:
            raise CacheError("NO_FREE_SLOT: every state slot is taken.")
        slot = self._free_slots.pop()
        self._live[request_id] = _Live(
            request_id, slot, tables=[BlockTable(size) for size in self.block_sizes]
        )
        for tensor in self.state_tensors:
            tensor[slot].zero_()
        return slot

    def release(self, request_id: str) -> None:
        """Give back everything the request holds: its pages of every group and its slot."""

        live = self._live.get(request_id)
        if live is None:
            raise CacheError(f"request {request_id!r} is not live.")
        if live.pending:
            raise CacheError(f"request {request_id!r} is part of an open step.")
        for allocator, table in zip(self.allocators, live.tables):
            pages = table.live_pages()
            if pages:
                allocator.release(pages)
        self._free_slots.append(live.state_slot)
        self._free_slots.sort(reverse=True)
        del self._live[request_id]

    def is_live(self, request_id: str) -> bool:
        return request_id in self._live

    def live_requests(self) -> tuple[str, ...]:
        return tuple(self._live)

    def committed_tokens(self, request_id: str) -> int:
        return self._live[request_id].committed

    def state_slot(self, request_id: str) -> int:
        return self._live[request_id].state_slot

    def block_table(self, request_id: str, group: int = 0) -> tuple[int, ...]:
        return self._live[request_id].tables[group].snapshot()

    # ---- the step transaction ---------------------------------------------------------
    def prepare_step(self, items: Sequence[StepItem]) -> StepReservation:
        if self._open is not None:
            raise CacheError("a step is already open; commit or abort it first.")
        seen: set[str] = set()
        for item in items:
            live = self._live.get(item.request_id)
            if live is None:
                raise CacheError(f"request {item.request_id!r} is not live.")
            if item.request_id in seen:
                raise CacheError(f"request {item.request_id!r} appears twice in one step.")
            seen.add(item.request_id)
            if item.start != live.committed:
                raise CacheError(
                    f"request {item.request_id!r}: the step starts at {item.start}, {live.committed} tokens are committed."
                )
            if item.end <= item.start or item.end > self.max_model_len:
                raise CacheError(f"request {item.request_id!r}: the step ends at {item.end} (limit {self.max_model_len}).")
        reservation = StepReservation(self._next_step_id)
        self._next_step_id += 1
        taken: list[tuple[int, list[int]]] = []
        try:
            for item in items:
                live = self._live[item.request_id]
                meta = SequenceStepMeta(item.request_id, live.state_slot, item.start, item.end, [], [], [])
                for index, (allocator, table) in enumerate(zip(self.allocators, live.tables)):
                    missing = table.pages_for(item.end) - len(table.pages)
                    new_pages = allocator.allocate(max(missing, 0))
                    taken.append((index, new_pages))
                    # without a new page the step reads the table's own snapshot, made once per change
                    tentative = tuple(table.pages + new_pages) if new_pages else table.snapshot()
                    block_size = self.block_sizes[index]
                    if item.end == item.start + 1:
                        logical, offset = divmod(item.start, block_size)
                        slots = (tentative[logical] * block_size + offset,)
                    else:
                        slots = tuple(
                            tentative[position // block_size] * block_size + position % block_size
                            for position in range(item.start, item.end)
                        )
                    meta.block_tables.append(tentative)
                    meta.slot_mappings.append(slots)
                    meta.new_pages.append(new_pages)
                reservation.sequences.append(meta)
        except OutOfPagesError:
            for index, pages in taken:
                if pages:
                    self.allocators[index].release(pages)
            raise
        for item in items:
            self._live[item.request_id].pending = True
        self._open = reservation
        self._keep_state(reservation)
        return reservation

    def _keep_state(self, reservation: StepReservation) -> None:
        """Per-request state is part of the transaction: the rows of the step's
        requests are copied before the step may write them (one small gather per state
        tensor, in stream order behind the step before), so that an aborted step, or
        the eager run before a recording, can be undone.  A model without state copies nothing."""

        if not self.state_tensors or not reservation.sequences:
            return
        import torch

        slots = torch.tensor([meta.state_slot for meta in reservation.sequences], dtype=torch.long,
                             device=self.state_tensors[0].device)
        reservation.state_before = [(slots, tensor.index_select(0, slots)) for tensor in self.state_tensors]

    def restore_state(self, reservation: StepReservation) -> None:
        """Puts the state of the step's requests back to what it was at ``prepare_step``."""

        for tensor, (slots, rows) in zip(self.state_tensors, reservation.state_before):
            tensor.index_copy_(0, slots, rows)

    def commit_step(self, reservation: StepReservation) -> None:
        self._close(reservation)
        reservation.state_before = []
        for meta in reservation.sequences:
            live = self._live[meta.request_id]
            for group, table, pages in zip(self.layout.groups, live.tables, meta.new_pages):
                table.extend(pages)
            live.committed = meta.after
            live.pending = False
            self._give_back_passed_pages(live)

    def abort_step(self, reservation: StepReservation) -> None:
        """Gives exactly the step's new pages back and restores the state of its
        requests; keys and values that the step wrote lie above the committed lengths
        and are never read."""

        self._close(reservation)
        self.restore_state(reservation)
        reservation.state_before = []
        for meta in reservation.sequences:
            for allocator, pages in zip(self.allocators, meta.new_pages):
                if pages:
                    allocator.release(pages)
            self._live[meta.request_id].pending = False

    def _close(self, reservation: StepReservation) -> None:
        if reservation.closed or self._open is not reservation:
            raise CacheError("this step is not the open one (a step id can be used once).")
        reservation.closed = True
        self._open = None

    def _give_back_passed_pages(self, live: _Live) -> None:
        """With ``n`` tokens committed the next query stands at ``n`` or later and
        reads keys ``>= n - window + 1``; pages wholly below that go back."""

        for group, allocator, table in zip(self.layout.groups, self.allocators, live.tables):
            if group.window is None:
                continue
            pages = table.give_back_before(live.committed - group.window + 1)
            if pages:
                allocator.release(pages)

    # ---- accounting -------------------------------------------------------------------
    def capacity(self) -> CapacitySnapshot:
        return CapacitySnapshot(
            block_sizes=self.block_sizes,
            total_blocks=self.num_blocks,
            free_blocks=tuple(allocator.free_count() for allocator in self.allocators),
            free_slots=len(self._free_slots),
            total_slots=self.max_num_seqs,
            held_blocks={
                request_id: tuple(table.live_count() for table in live.tables)
                for request_id, live in self._live.items()
            },
            windows=tuple(group.window for group in self.layout.groups),
        )

    def assert_invariants(self) -> None:
        """No page is lost or held twice: per group, the pages of all tables, the
        open step's tentative pages and the free list are disjoint and add up."""

        for index, allocator in enumerate(self.allocators):
            allocator.assert_invariants()
            held: list[int] = []
            for live in self._live.values():
                held.extend(live.tables[index].live_pages())
            if self._open is not None:
                for meta in self._open.sequences:
                    held.extend(meta.new_pages[index])
            if len(held) != len(set(held)):
                raise AssertionError(f"group {index}: a page is held twice.")
            if set(held) & set(allocator.free_ids()):
                raise AssertionError(f"group {index}: a held page is on the free list.")
            if len(held) + allocator.free_count() != allocator.num_pages:
                raise AssertionError(f"group {index}: pages are lost ({len(held)} held, {allocator.free_count()} free).")
        slots = [live.state_slot for live in self._live.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise AssertionError("a state slot is held twice.")
        if len(slots) + len(self._free_slots) != self.max_num_seqs:
            raise AssertionError("state slots are lost.")
