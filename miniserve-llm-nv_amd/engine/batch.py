"""From (request, its next tokens) to the flat tensors of one step.

The reference builds one tensor set per prefill request and one flat set for the
decode rows (miniserve/engine/batch_builder.py:128-248, flat_batch.py:355-487);
here there is one flat ragged batch for everything.  The host check that every
slot agrees with its block table (reference: flat_batch.py:296-333) is kept: it
is cheap and stops an allocator fault before a kernel can scribble.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import torch

from ..cache.manager import StepReservation
from ..parts.base import GroupStepView, QueryTiles, StepContext


QUERY_TILE = 64     # tokens of one sequence that one workgroup of the tiled attention kernel serves


@dataclass(frozen=True)
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request_id: str
    token_ids: tuple[int, ...]
    want: tuple[int, ...] = ()

    def __post_init__(self) -> None:
        if not self.token_ids:
            raise ValueError(f"entry {self.request_id!r} brings no tokens.")
        if any(not isinstance(t, int) or isinstance(t, bool) or t < 0 for t in self.token_ids):
            raise ValueError(f"entry {self.request_id!r}: token ids must be non-negative integers.")
        if any(not isinstance(w, int) or isinstance(w, bool) or not 0 <= w < len(self.token_ids) for w in self.want):
            raise ValueError(f"entry {self.request_id!r}: wanted places must index its tokens.")


def build_step_context(
    entries: Sequence[StepEntry],
    reservation: StepReservation,
    *,
    block_size: int,
    pool_pages: Sequence[int],
    vocab_size: int,
    device: torch.device | str,
) -> tuple[StepContext, torch.Tensor | None]:
    """All integer metadata of the step is packed into one host buffer and sent to
    the device in one copy; the context's tensors are views of it."""

    if len(entries) != len(reservation.sequences):
        raise ValueError("entries and reservation disagree.")
    # Sequences that bring one token are laid out first; the logits keep the order of
    # the entries as given.
    layout = sorted(range(len(entries)), key=lambda i: len(entries[i].token_ids) != 1)
    decode_prefix = sum(1 for entry in entries if len(entry.token_ids) == 1)
    base_of_entry = [0] * len(entries)
    token_ids: list[int] = []
    positions: list[int] = []
    seq_of_token: list[int] = []
    query_start = [0]
    context_lens: list[int] = []
    state_slots: list[int] = []
    logit_rows: list[int] = []
    query_lens: list[int] = []
    first_positions: list[int] = []
    num_groups = len(pool_pages)
    slot_mappings: list[list[int]] = [[] for _ in range(num_groups)]
    widest = [1] * num_groups

    tile_seq: list[int] = []
    tile_token: list[int] = []
    tile_length: list[int] = []
    metas_in_layout = [reservation.sequences[i] for i in layout]
    for index, original in enumerate(layout):
        entry, meta = entries[original], reservation.sequences[original]
        if entry.request_id != meta.request_id or len(entry.token_ids) != meta.after - meta.before:
            raise ValueError(f"entry {entry.request_id!r} does not match its reservation.")
        if any(token >= vocab_size for token in entry.token_ids):
            raise ValueError(f"entry {entry.request_id!r}: a token id is outside the vocabulary of {vocab_size}.")
        base = len(token_ids)
        base_of_entry[original] = base
        if index >= decode_prefix:
            for start in range(0, len(entry.token_ids), QUERY_TILE):
                tile_seq.append(index)
                tile_token.append(base + start)
                tile_length.append(min(QUERY_TILE, len(entry.token_ids) - start))
        token_ids.extend(entry.token_ids)
        positions.extend(range(meta.before, meta.after))
        seq_of_token.extend([index] * len(entry.token_ids))
        query_start.append(len(token_ids))
        context_lens.append(meta.after)
        state_slots.append(meta.state_slot)
        query_lens.append(len(entry.token_ids))
        first_positions.append(meta.before)
        for group in range(num_groups):
            table = meta.block_tables[group]
            slots = meta.slot_mappings[group]
            # slot == table[pos // bs] * bs + pos % bs, and the page lies in the pool
            for position, slot in zip(range(meta.before, meta.after), slots):
                page = table[position // block_size]
                if not 0 <= page < pool_pages[group] or slot != page * block_size + position % block_size:
                    raise RuntimeError(f"request {entry.request_id!r}: slot {slot} disagrees with its block table.")
            slot_mappings[group].extend(slots)
            widest[group] = max(widest[group], len(table))

    for original, entry in enumerate(entries):
        logit_rows.extend(base_of_entry[original] + place for place in entry.want)

    n, s = len(token_ids), len(entries)
    packed: list[int] = []
    offsets: dict[str, tuple[int, int]] = {}

    def put(name: str, values: Sequence[int]) -> None:
        offsets[name] = (len(packed), len(values))
        packed.extend(values)

    put("token_ids", token_ids)
    put("positions", positions)
    put("seq_of_token", seq_of_token)
    put("query_start", query_start)
    put("context_lens", context_lens)
    put("state_slots", state_slots)
    put("logit_rows", logit_rows)
    put("tile_seq", tile_seq)
    put("tile_token", tile_token)
    put("tile_length", tile_length)
    for group in range(num_groups):
        put(f"slots{group}", slot_mappings[group])
        flat: list[int] = []
        for meta in metas_in_layout:
            table = meta.block_tables[group]
            # a page that was given back is never read; 0 keeps the entry inside the pool
            flat.extend(page if page >= 0 else 0 for page in table)
            flat.extend([0] * (widest[group] - len(table)))
        put(f"table{group}", flat)

    host = torch.tensor(packed, dtype=torch.int32)
    if torch.device(device).type == "cuda":
        host = host.pin_memory()
    buffer = host.to(device, non_blocking=True)

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
        tiles=QueryTiles(len(tile_seq), view("tile_seq"), view("tile_token"), view("tile_length")) if tile_seq else None,
    )
    rows = view("logit_rows") if logit_rows else None
    return ctx, rows
