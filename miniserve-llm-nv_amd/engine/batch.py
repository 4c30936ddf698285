"""From (request, its next tokens) to the flat tensors of one step.

The reference builds one tensor set per prefill request and one flat set for the
decode rows (miniserve/engine/batch_builder.py:128-248, flat_batch.py:355-487);
here there is one flat ragged batch for everything.  The host check that every
slot agrees with its block table (reference: flat_batch.py:296-333) is kept: it
is cheap and stops an allocator fault before a kernel can scribble.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Mapping, Sequence

import numpy as np
import torch

from ..cache.manager import StepReservation
from ..parts.base import GroupStepView, HostBatch, StepContext


@dataclass(frozen=True)
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request_id: str
    token_ids: tuple[int, ...]
    want: tuple[int, ...] = ()

    def __post_init__(self) -> None:
        tokens, want = self.token_ids, self.want
        if len(tokens) == 1 and type(tokens[0]) is int and tokens[0] >= 0 and (want == (0,) or want == ()):
            return          # a decoded token: the common case, checked without loops
        if not self.token_ids:
            raise ValueError(f"entry {self.request_id!r} brings no tokens.")
        # a portion of a prompt has hundreds of tokens: their types and their least are taken
        # without a Python-level loop (a bool is an int to isinstance, not to type)
        if set(map(type, self.token_ids)) != {int} or min(self.token_ids) < 0:
            raise ValueError(f"entry {self.request_id!r}: token ids must be non-negative integers.")
        if any(not isinstance(w, int) or isinstance(w, bool) or not 0 <= w < len(self.token_ids) for w in self.want):
            raise ValueError(f"entry {self.request_id!r}: wanted places must index its tokens.")


@dataclass
class BuiltStep:
    """A step's tensors, made but not yet sent: the context's tensors are views of
    ``buffer``, which holds nothing before :meth:`send`.  Token ids of entries that
    bring one token may still be set until then."""

    ctx: StepContext
    rows: torch.Tensor | None
    request_ids: tuple[str, ...]
    query_lens_of_entries: tuple[int, ...]
    vocab_size: int
    _host: torch.Tensor
    _buffer: torch.Tensor
    _token_places: tuple[int, ...]        # of each entry's first token, in the host buffer
    _sent: bool = False

    def set_single_token(self, entry_index: int, token: int) -> None:
        if self._sent or self.query_lens_of_entries[entry_index] != 1:
            raise RuntimeError("only a single token of a step that is not sent yet can be set.")
        if not 0 <= token < self.vocab_size:
            raise ValueError(
                f"entry {self.request_ids[entry_index]!r}: a token id is outside the vocabulary of {self.vocab_size}."
            )
        self._host[self._token_places[entry_index]] = token

    def send(self) -> None:
        if self._sent:
            raise RuntimeError("the step was sent already.")
        if self._buffer is not self._host:
            self._buffer.copy_(self._host, non_blocking=True)
        self._sent = True


def build_step(
    entries: Sequence[StepEntry],
    reservation: StepReservation,
    *,
    block_sizes: Sequence[int],
    pool_pages: Sequence[int],
    vocab_size: int,
    device: torch.device | str,
    step_tables: Callable[[HostBatch], Mapping[str, Sequence[int]]] | None = None,
) -> BuiltStep:
    """All integer metadata of the step is packed into one host buffer that goes to
    the device in one copy (:meth:`BuiltStep.send`); the context's tensors are views
    of the device buffer.  ``step_tables``: the model's hook that makes the integer
    tables its parts want for this batch (tile lists of a kernel, say); they are
    packed into the same buffer and handed to the parts as ``ctx.tables``."""

    if len(entries) != len(reservation.sequences):
        raise ValueError("entries and reservation disagree.")
    # Sequences that bring one token are laid out first; the logits keep the order of
    # the entries as given.
    layout = sorted(range(len(entries)), key=lambda i: len(entries[i].token_ids) != 1)
    decode_prefix = sum(1 for entry in entries if len(entry.token_ids) == 1)
    metas_in_layout = [reservation.sequences[i] for i in layout]
    num_groups = len(pool_pages)
    s = len(entries)
    query_lens = [len(entries[original].token_ids) for original in layout]
    n = sum(query_lens)
    query_start = [0] * (s + 1)
    for index, length in enumerate(query_lens):
        query_start[index + 1] = query_start[index] + length
    first_positions = [meta.before for meta in metas_in_layout]
    part_tables: dict[str, np.ndarray] = {}
    if step_tables is not None:
        host_batch = HostBatch(tuple(query_lens), tuple(query_start), tuple(first_positions), decode_prefix)
        for name, values in step_tables(host_batch).items():
            part_tables[name] = np.asarray(values, dtype=np.int64)
            if part_tables[name].ndim != 1 or (part_tables[name].size and (
                    part_tables[name].min() < -(2**31) or part_tables[name].max() >= 2**31)):
                raise ValueError(f"step table {name!r} must be a list of 32-bit integers.")
    num_rows = sum(len(entry.want) for entry in entries)
    widest = [max(1, max(len(meta.block_tables[group]) for meta in metas_in_layout)) for group in range(num_groups)]

    offsets: dict[str, tuple[int, int]] = {}
    total = 0
    sizes = [("token_ids", n), ("positions", n), ("seq_of_token", n), ("query_start", s + 1), ("context_lens", s),
             ("state_slots", s), ("logit_rows", num_rows)]
    sizes += [(f"part:{name}", values.size) for name, values in part_tables.items()]
    for group in range(num_groups):
        sizes += [(f"slots{group}", n), (f"table{group}", s * widest[group])]
    for name, size in sizes:
        offsets[name] = (total, size)
        total += size
    on_gpu = torch.device(device).type == "cuda"
    host = torch.empty(total, dtype=torch.int32, pin_memory=on_gpu)
    numbers = host.numpy()

    def region(name: str) -> np.ndarray:
        start, size = offsets[name]
        return numbers[start : start + size]

    token_ids, positions, seq_of_token = region("token_ids"), region("positions"), region("seq_of_token")
    slot_regions = [region(f"slots{group}") for group in range(num_groups)]
    table_regions = [region(f"table{group}") for group in range(num_groups)]
    for table_region in table_regions:
        table_region[:] = 0
    context_lens = [meta.after for meta in metas_in_layout]
    state_slots = [meta.state_slot for meta in metas_in_layout]
    base_of_entry = [0] * s

    for index, original in enumerate(layout):
        entry, meta = entries[original], metas_in_layout[index]
        length = query_lens[index]
        if entry.request_id != meta.request_id or length != meta.after - meta.before:
            raise ValueError(f"entry {entry.request_id!r} does not match its reservation.")
        base = query_start[index]
        base_of_entry[original] = base
        if length == 1:
            # one token: plain integers (an array per row would cost more than it saves)
            token = entry.token_ids[0]
            if token >= vocab_size:
                raise ValueError(f"entry {entry.request_id!r}: a token id is outside the vocabulary of {vocab_size}.")
            token_ids[base] = token
            positions[base] = meta.before
            seq_of_token[base] = index
            for group in range(num_groups):
                block_size = block_sizes[group]
                logical, offset = divmod(meta.before, block_size)
                table = meta.block_tables[group]
                slot = meta.slot_mappings[group][0]
                page = table[logical]
                # slot == table[pos // bs] * bs + pos % bs, and the page lies in the pool
                if not 0 <= page < pool_pages[group] or slot != page * block_size + offset:
                    raise RuntimeError(f"request {entry.request_id!r}: slot {slot} disagrees with its block table.")
                slot_regions[group][base] = slot
                start = index * widest[group]
                table_regions[group][start : start + len(table)] = table
            continue
        tokens = np.asarray(entry.token_ids, dtype=np.int64)
        if int(tokens.max()) >= vocab_size:
            raise ValueError(f"entry {entry.request_id!r}: a token id is outside the vocabulary of {vocab_size}.")
        token_ids[base : base + length] = tokens
        run = np.arange(meta.before, meta.after, dtype=np.int64)
        positions[base : base + length] = run
        seq_of_token[base : base + length] = index
        for group in range(num_groups):
            block_size = block_sizes[group]
            logical, offset = np.divmod(run, block_size)
            table = np.asarray(meta.block_tables[group], dtype=np.int64)
            slots = np.asarray(meta.slot_mappings[group], dtype=np.int64)
            pages = table[logical]
            agree = (pages >= 0) & (pages < pool_pages[group]) & (slots == pages * block_size + offset)
            if not bool(agree.all()):
                slot = int(slots[int(np.argmin(agree))])
                raise RuntimeError(f"request {entry.request_id!r}: slot {slot} disagrees with its block table.")
            slot_regions[group][base : base + length] = slots
            start = index * widest[group]
            table_regions[group][start : start + len(table)] = table
    for table_region in table_regions:
        # a page that was given back is never read; 0 keeps the entry inside the pool
        np.maximum(table_region, 0, out=table_region)

    logit_rows: list[int] = []
    for original, entry in enumerate(entries):
        logit_rows.extend(base_of_entry[original] + place for place in entry.want)
    region("query_start")[:] = query_start
    region("context_lens")[:] = context_lens
    region("state_slots")[:] = state_slots
    region("logit_rows")[:] = logit_rows
    for name, values in part_tables.items():
        region(f"part:{name}")[:] = values
    buffer = torch.empty(total, dtype=torch.int32, device=device) if on_gpu else host

    def view(name: str) -> torch.Tensor:
        start, length = offsets[name]
        return buffer[start : start + length]

    groups = [
        GroupStepView(block_table=view(f"table{g}").view(s, widest[g]), slot_mapping=view(f"slots{g}"))
        for g in range(num_groups)
    ]
    ctx = StepContext(
        num_tokens=n,
        num_seqs=s,
        token_ids=view("token_ids"),
        positions=view("positions"),
        seq_of_token=view("seq_of_token"),
        query_start=view("query_start"),
        context_lens=view("context_lens"),
        state_slots=view("state_slots"),
        groups=groups,
        query_lens=query_lens,
        context_lens_host=context_lens,
        query_start_host=query_start,
        state_slots_host=state_slots,
        first_positions_host=first_positions,
        decode_prefix=decode_prefix,
        tables={name: view(f"part:{name}") for name in part_tables},
    )
    rows = view("logit_rows") if logit_rows else None
    token_start = offsets["token_ids"][0]
    return BuiltStep(
        ctx=ctx,
        rows=rows,
        request_ids=tuple(entry.request_id for entry in entries),
        query_lens_of_entries=tuple(len(entry.token_ids) for entry in entries),
        vocab_size=vocab_size,
        _host=host,
        _buffer=buffer,
        _token_places=tuple(token_start + base for base in base_of_entry),
    )
