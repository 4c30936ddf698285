"""The step's integer tensors as the batch builder packs them, against a real cache
manager, on the CPU: layout (single tokens first), positions, slots, block tables,
the rows of the wanted logits, the tables that parts ask for, and what it refuses."""

from __future__ import annotations

from types import SimpleNamespace

import pytest
import torch

from miniserve_amd.cache import CacheLayout, CacheManager, StepItem
from miniserve_amd.engine.batch import StepEntry, build_step
from miniserve_amd.parts import KVCacheNeed

BLOCK = 4
VOCAB = 50


def make_cache(blocks=16, window=None):
    needs = [SimpleNamespace(call=0, need=KVCacheNeed(1, 8), cache_from=None)]
    if window is not None:
        needs.append(SimpleNamespace(call=1, need=KVCacheNeed(1, 8, window=window), cache_from=None))
    return CacheManager(CacheLayout.from_needs(needs), block_size=BLOCK, num_blocks=blocks, max_num_seqs=4, max_model_len=64)


def run(cache, entries):
    items = [StepItem(e.request_id, cache.committed_tokens(e.request_id), cache.committed_tokens(e.request_id) + len(e.token_ids))
             for e in entries]
    return cache.prepare_step(items)


def built(cache, entries, reservation, **more):
    return build_step(entries, reservation, block_sizes=cache.block_sizes, pool_pages=cache.num_blocks,
                      vocab_size=VOCAB, device="cpu", **more)


def test_layout_positions_slots_tables_and_rows():
    cache = make_cache()
    for name in ("a", "b", "c"):
        cache.admit(name)
    # a has 6 tokens and b 9 in the cache already
    first = [StepEntry("a", tuple(range(6))), StepEntry("b", tuple(range(10, 19)))]
    cache.commit_step(run(cache, first))
    # the step: c brings a portion of 5 (places 1 and 4 wanted), a one token, b one token: given in this order
    entries = [StepEntry("c", (1, 2, 3, 4, 5), (1, 4)), StepEntry("a", (7,), (0,)), StepEntry("b", (8,), (0,))]
    reservation = run(cache, entries)
    step = built(cache, entries, reservation)
    ctx = step.ctx
    # single tokens first, in their given order, then the portion
    assert ctx.decode_prefix == 2 and ctx.num_seqs == 3 and ctx.num_tokens == 7
    assert ctx.query_lens == [1, 1, 5] and ctx.query_start.tolist() == [0, 1, 2, 7]
    assert ctx.token_ids.tolist() == [7, 8, 1, 2, 3, 4, 5]
    assert ctx.positions.tolist() == [6, 9, 0, 1, 2, 3, 4]
    assert ctx.seq_of_token.tolist() == [0, 1, 2, 2, 2, 2, 2]
    assert ctx.context_lens.tolist() == [7, 10, 5] and ctx.first_positions_host == [6, 9, 0]
    # the wanted rows keep the order of the entries as given: c's two places, then a, then b
    assert step.rows.tolist() == [2 + 1, 2 + 4, 0, 1]
    # every slot is its page times the page size plus the place in the page; tables are as wide as the longest
    table = ctx.groups[0].block_table
    assert tuple(table.shape) == (3, 3)
    for token in range(ctx.num_tokens):
        row, position = int(ctx.seq_of_token[token]), int(ctx.positions[token])
        assert int(ctx.groups[0].slot_mapping[token]) == int(table[row, position // BLOCK]) * BLOCK + position % BLOCK
    pages = [page for row, used in zip(table.tolist(), (2, 3, 2)) for page in row[:used]]
    assert len(set(pages)) == len(pages)                                  # no page in two tables
    assert table[0, 2] == 0                                               # beyond a table's end: 0, inside the pool
    # state slots are the requests' own, in layout order
    assert ctx.state_slots.tolist() == [reservation.sequences[i].state_slot for i in (1, 2, 0)]
    # a single token may still be set before the step is sent, others not
    step.set_single_token(1, 33)
    assert ctx.token_ids.tolist()[0] == 33
    with pytest.raises(RuntimeError):
        step.set_single_token(0, 3)
    with pytest.raises(ValueError, match="vocabulary"):
        step.set_single_token(1, VOCAB)
    step.send()
    with pytest.raises(RuntimeError):
        step.set_single_token(1, 2)
    cache.commit_step(reservation)
    cache.assert_invariants()


def test_two_groups_have_tables_and_slots_of_their_own():
    cache = make_cache(window=6)
    cache.admit("a")
    reservation = run(cache, [StepEntry("a", tuple(range(11)))])
    entries = [StepEntry("a", tuple(range(11)), (10,))]
    step = built(cache, entries, reservation)
    assert len(step.ctx.groups) == 2
    for group in step.ctx.groups:
        table = group.block_table
        for token in range(11):
            assert int(group.slot_mapping[token]) == int(table[0, token // BLOCK]) * BLOCK + token % BLOCK
    cache.commit_step(reservation)
    # once the window has passed a page it is given back: the next step's table holds 0 there, never a stale page
    cache.commit_step(run(cache, [StepEntry("a", (1,))]))
    reservation = run(cache, [StepEntry("a", (2,), (0,))])
    step = built(cache, [StepEntry("a", (2,), (0,))], reservation)
    kept = reservation.sequences[0].block_tables
    assert kept[0] == (0, 1, 2, 3) and kept[1] == (-1, 1, 2, 0)            # the page that was given back is used again, as the newest
    assert step.ctx.groups[0].block_table[0].tolist() == [0, 1, 2, 3]
    assert step.ctx.groups[1].block_table[0].tolist() == [0, 1, 2, 0]       # (-1 becomes 0: never read, inside the pool)
    assert int(step.ctx.groups[1].slot_mapping[0]) == 0 * BLOCK + 12 % BLOCK
    cache.abort_step(reservation)
    cache.assert_invariants()


def test_tables_that_parts_ask_for_travel_with_the_step():
    cache = make_cache()
    cache.admit("a")
    cache.admit("b")
    entries = [StepEntry("a", (1, 2, 3)), StepEntry("b", (4,))]
    reservation = run(cache, entries)
    seen = []

    def step_tables(batch):
        seen.append(batch)
        return {"toy.rows": [length for length in batch.query_lens], "toy.none": []}

    step = built(cache, entries, reservation, step_tables=step_tables)
    assert seen[0].query_lens == (1, 3) and seen[0].query_start == (0, 1, 4) and seen[0].first_positions == (0, 0)
    assert seen[0].decode_prefix == 1
    assert step.ctx.tables["toy.rows"].tolist() == [1, 3] and step.ctx.tables["toy.none"].numel() == 0
    assert step.ctx.tables["toy.rows"].dtype == torch.int32
    with pytest.raises(ValueError, match="32-bit"):
        built(cache, entries, reservation, step_tables=lambda batch: {"toy.big": [2**31]})
    cache.abort_step(reservation)


def test_what_the_builder_refuses():
    cache = make_cache()
    cache.admit("a")
    entries = [StepEntry("a", (1, 2, 3))]
    reservation = run(cache, entries)
    with pytest.raises(ValueError, match="vocabulary"):
        built(cache, [StepEntry("a", (1, VOCAB, 3))], reservation)
    with pytest.raises(ValueError, match="reservation"):
        built(cache, [StepEntry("a", (1, 2))], reservation)                # another length than was reserved
    with pytest.raises(ValueError, match="disagree"):
        built(cache, entries + [StepEntry("b", (1,))], reservation)
    # a slot that is not where its block table says: refused before anything reaches a kernel
    meta = reservation.sequences[0]
    wrong = list(meta.slot_mappings[0])
    wrong[1] += BLOCK
    broken = SimpleNamespace(sequences=[SimpleNamespace(
        request_id=meta.request_id, before=meta.before, after=meta.after, state_slot=meta.state_slot,
        block_tables=meta.block_tables, slot_mappings=[wrong])])
    with pytest.raises(RuntimeError, match="disagrees with its block table"):
        built(cache, entries, broken)
    cache.abort_step(reservation)
    for bad in ((), (1.0,), (True,), (-1,)):
        with pytest.raises(ValueError):
            StepEntry("a", bad)
    with pytest.raises(ValueError, match="wanted places"):
        StepEntry("a", (1, 2), (2,))
