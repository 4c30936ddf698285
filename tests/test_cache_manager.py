"""Allocator, block tables, cache groups, state slots and the step transaction (no GPU)."""

from __future__ import annotations

import random
from dataclasses import dataclass

import pytest

from miniserve_amd.cache import (
    RETURNED,
    BlockTable,
    CacheError,
    CacheLayout,
    CacheManager,
    OutOfPagesError,
    PageAllocator,
    StepItem,
)
from miniserve_amd.parts import KVCacheNeed, StateNeed


@dataclass
class Need:
    call: int
    need: object
    cache_from: int | None = None


def manager(needs=None, *, block_size=4, num_blocks=8, slots=4, max_len=256) -> CacheManager:
    needs = needs or [Need(0, KVCacheNeed(2, 64))]
    return CacheManager(
        CacheLayout.from_needs(needs), block_size=block_size, num_blocks=num_blocks, max_num_seqs=slots,
        max_model_len=max_len,
    )


# ---- allocator and table: the reference's own vectors ---------------------------------

def test_allocate_retain_release_and_total_conservation():
    # reference: tests/unit/test_block_allocator.py:13-23
    allocator = PageAllocator(6)
    blocks = allocator.allocate(2)
    assert blocks == [0, 1]
    allocator.retain(blocks)
    assert [allocator.refcount(b) for b in blocks] == [2, 2]
    allocator.release(blocks)
    assert allocator.free_count() == 4
    allocator.release(blocks)
    assert allocator.free_count() == 6
    allocator.assert_invariants()


def test_out_of_pages_and_invalid_release_are_atomic():
    # reference: tests/unit/test_block_allocator.py:26-37
    allocator = PageAllocator(3)
    allocator.allocate(2)
    state = lambda: (allocator.free_ids(), [allocator.refcount(page) for page in range(3)])
    before = state()
    with pytest.raises(OutOfPagesError, match="2 asked for, 1 of 3 free"):
        allocator.allocate(2)
    assert state() == before
    with pytest.raises(RuntimeError, match="they are free"):
        allocator.release((0, 2))           # page 0 is held, page 2 is not: neither changes
    assert state() == before
    with pytest.raises(ValueError, match="named twice"):
        allocator.release((0, 0))
    with pytest.raises(IndexError):
        allocator.release((3,))
    with pytest.raises(TypeError):
        allocator.release((True,))
    assert state() == before
    allocator.assert_invariants()


def test_lowest_id_first_after_release():
    allocator = PageAllocator(5)
    allocator.allocate(5)
    allocator.release([3, 1])
    assert allocator.allocate(2) == [1, 3]


@pytest.mark.parametrize("value", [True, 1.5, "2", -1])
def test_allocator_rejects_coercible_or_invalid_counts(value):
    with pytest.raises((TypeError, ValueError)):
        PageAllocator(value)
    with pytest.raises(ValueError, match="whole number"):
        PageAllocator(2).allocate(value)


@pytest.mark.parametrize(
    ("position", "expected"),
    [(0, (0, 5, 0)), (15, (0, 5, 15)), (16, (1, 2, 0)), (17, (1, 2, 1)), (31, (1, 2, 15)), (32, (2, 7, 0)), (33, (2, 7, 1))],
)
def test_noncontiguous_block_table_boundaries(position, expected):
    # reference: tests/unit/test_block_allocator.py:66-81
    table = BlockTable(16, [5, 2, 7])
    assert table.locate(position) == expected
    assert table.slot(position) == expected[1] * 16 + expected[2]


def test_block_table_rejects_invalid_metadata():
    for block_size, ids in ((True, [0]), (16, [-1]), (16, [True]), (16, [1.5]), (16, [3, 3])):
        with pytest.raises(ValueError):
            BlockTable(block_size, ids)
    table = BlockTable(16, [0])
    with pytest.raises(ValueError):
        table.extend([True])
    with pytest.raises(ValueError):
        table.extend([0])
    with pytest.raises(ValueError):
        table.locate(1.5)
    with pytest.raises(IndexError):
        table.locate(16)


def test_window_table_gives_pages_back():
    table = BlockTable(4, [9, 8, 7, 6])
    assert table.give_back_before(3) == []
    assert table.give_back_before(9) == [9, 8]
    assert table.snapshot() == (RETURNED, RETURNED, 7, 6) and table.live_pages() == [7, 6]
    with pytest.raises(IndexError, match="given back"):
        table.locate(5)
    assert table.give_back_before(8) == []
    table.extend([9])
    assert table.slot(16) == 9 * 4


def test_the_snapshot_is_one_object_until_the_table_changes():
    table = BlockTable(4, [3, 5])
    first = table.snapshot()
    assert first == (3, 5) and table.snapshot() is first
    table.extend([])
    assert table.snapshot() is first and table.live_count() == 2
    table.extend([7])
    assert table.snapshot() == (3, 5, 7) and table.snapshot() is not first
    kept = table.snapshot()
    assert table.give_back_before(3) == [] and table.snapshot() is kept
    assert table.give_back_before(4) == [3] and table.snapshot() == (RETURNED, 5, 7) and table.live_count() == 2


def test_a_step_without_a_new_page_shares_the_table_snapshot():
    m = manager()
    m.admit("r")
    m.commit_step(m.prepare_step([StepItem("r", 0, 5)]))
    one = m.prepare_step([StepItem("r", 5, 6)])
    table = one.sequences[0].block_tables[0]
    assert one.sequences[0].new_pages[0] == [] and one.sequences[0].slot_mappings[0] == (table[1] * 4 + 1,)
    m.commit_step(one)
    two = m.prepare_step([StepItem("r", 6, 7)])
    assert two.sequences[0].block_tables[0] is table          # nothing changed: the same object
    m.commit_step(two)
    three = m.prepare_step([StepItem("r", 7, 9)])              # crosses into a third page
    assert len(three.sequences[0].new_pages[0]) == 1 and len(three.sequences[0].block_tables[0]) == 3
    m.abort_step(three)
    assert m.prepare_step([StepItem("r", 7, 8)]).sequences[0].block_tables[0] is table


# ---- the manager ------------------------------------------------------------------------

def test_ten_tokens_take_three_pages_and_abort_restores():
    # reference: tests/unit/test_kv_capacity_accounting.py:38-75 (bs 4, 8 blocks)
    m = manager()
    m.admit("r")
    step = m.prepare_step([StepItem("r", 0, 10)])
    meta = step.sequences[0]
    assert meta.block_tables[0] == (0, 1, 2) and meta.new_pages[0] == [0, 1, 2]
    assert meta.slot_mappings[0] == tuple(range(10))
    assert m.capacity().free_blocks == (5,)
    m.abort_step(step)
    assert m.capacity().free_blocks == (8,) and m.committed_tokens("r") == 0
    step = m.prepare_step([StepItem("r", 0, 10)])
    m.commit_step(step)
    assert m.committed_tokens("r") == 10 and m.block_table("r") == (0, 1, 2)
    step = m.prepare_step([StepItem("r", 10, 13)])     # 2 slots left in page 2, then a new page
    assert step.sequences[0].slot_mappings[0] == (10, 11, 12)
    assert step.sequences[0].new_pages[0] == [3]
    m.commit_step(step)
    m.release("r")
    assert m.capacity().free_blocks == (8,) and m.capacity().free_slots == 4
    m.assert_invariants()


def test_step_rules():
    m = manager()
    m.admit("a")
    with pytest.raises(CacheError, match="already live"):
        m.admit("a")
    with pytest.raises(CacheError, match="not live"):
        m.prepare_step([StepItem("b", 0, 1)])
    with pytest.raises(CacheError, match="starts at 3"):
        m.prepare_step([StepItem("a", 3, 4)])
    with pytest.raises(CacheError, match="twice"):
        m.prepare_step([StepItem("a", 0, 1), StepItem("a", 0, 1)])
    with pytest.raises(CacheError, match="limit 256"):
        m.prepare_step([StepItem("a", 0, 257)])
    step = m.prepare_step([StepItem("a", 0, 5)])
    with pytest.raises(CacheError, match="already open"):
        m.prepare_step([StepItem("a", 0, 5)])
    with pytest.raises(CacheError, match="open step"):
        m.release("a")
    m.commit_step(step)
    with pytest.raises(CacheError, match="used once"):
        m.commit_step(step)
    with pytest.raises(CacheError, match="used once"):
        m.abort_step(step)


def test_out_of_pages_in_prepare_leaves_no_trace():
    m = manager(num_blocks=4)
    m.admit("a")
    m.admit("b")
    m.commit_step(m.prepare_step([StepItem("a", 0, 9)]))        # 3 pages
    with pytest.raises(OutOfPagesError):
        m.prepare_step([StepItem("a", 9, 12), StepItem("b", 0, 8)])   # 0 + 2 pages, 1 free
    assert m.capacity().free_blocks == (1,)
    m.assert_invariants()
    m.commit_step(m.prepare_step([StepItem("b", 0, 4)]))
    m.assert_invariants()


def test_state_slots_are_numbered_and_reused():
    m = manager(slots=2)
    assert m.admit("a") == 0 and m.admit("b") == 1
    with pytest.raises(CacheError, match="NO_FREE_SLOT"):
        m.admit("c")
    m.release("a")
    assert m.admit("c") == 0
    m.assert_invariants()


def test_groups_by_need_shared_caches_and_state():
    full, window, state = KVCacheNeed(2, 16), KVCacheNeed(2, 16, window=6), StateNeed((5,))
    needs = [Need(0, full), Need(1, window), Need(2, state), Need(3, full), Need(4, full, cache_from=0), Need(5, None)]
    layout = CacheLayout.from_needs(needs)
    assert [g.calls for g in layout.groups] == [[0, 3], [1]]
    assert [(p.kind, p.group, p.index, p.write) for p in layout.placements] == [
        ("kv", 0, 0, True), ("kv", 1, 0, True), ("state", -1, 0, True), ("kv", 0, 1, True), ("kv", 0, 0, False),
        ("none", -1, -1, True),
    ]
    assert layout.bytes_per_token(2) == 2 * 2 * 2 * 16 * 2 + 2 * 1 * 2 * 16 * 2
    with pytest.raises(ValueError, match="owns none"):
        CacheLayout.from_needs([Need(0, state), Need(1, full, cache_from=0)])


def test_window_group_gives_pages_back_while_the_request_lives():
    needs = [Need(0, KVCacheNeed(1, 16)), Need(1, KVCacheNeed(1, 16, window=6))]
    m = manager(needs, block_size=4, num_blocks=[16, 4])
    m.admit("r")
    length = 0
    for portion in (5, 3, 1, 1, 6, 1, 1, 1, 2, 1):
        step = m.prepare_step([StepItem("r", length, length + portion)])
        m.commit_step(step)
        length += portion
        m.assert_invariants()
        full_table, window_table = m.block_table("r", 0), m.block_table("r", 1)
        assert len(full_table) == -(-length // 4) and RETURNED not in full_table
        # keys >= length - 6 + 1 must still be there; pages wholly below are gone
        first_needed = max(length - 6 + 1, 0) // 4
        assert all(page == RETURNED for page in window_table[:first_needed])
        assert all(page != RETURNED for page in window_table[first_needed:])
        assert m.capacity().free_blocks[1] == 4 - (len(window_table) - first_needed)
    assert length == 22                     # 6 pages of history passed through a pool of 4
    m.release("r")
    assert m.capacity().free_blocks == (16, 4)


def test_groups_with_page_sizes_of_their_own():
    """A mixer may ask for pages of another size than the engine's: its group has its
    own pool, tables and slots; one number of pages for the engine means as many tokens
    in every group."""

    needs = [Need(0, KVCacheNeed(1, 16)), Need(1, KVCacheNeed(1, 16, window=6, block_size=2)), Need(2, KVCacheNeed(1, 16))]
    m = manager(needs, block_size=8, num_blocks=6, max_len=64)
    assert m.block_sizes == (8, 2) and m.num_blocks == (6, 24)          # 48 tokens each
    assert [g.calls for g in m.layout.groups] == [[0, 2], [1]]
    capacity = m.capacity()
    assert capacity.block_sizes == (8, 2) and capacity.pages_for(0, 9) == (2, 5) and capacity.pages_for(9, 10) == (0, 0)
    assert capacity.most_pages_held(40, 1) == (5, 4) and capacity.room_for(9, (1, 1)) == 3     # 1 + 2 in the small pages
    m.admit("r")
    step = m.prepare_step([StepItem("r", 0, 11)])
    meta = step.sequences[0]
    assert [len(table) for table in meta.block_tables] == [2, 6]
    for group, size in enumerate((8, 2)):
        assert list(meta.slot_mappings[group]) == [
            meta.block_tables[group][position // size] * size + position % size for position in range(11)
        ]
    m.commit_step(step)
    m.assert_invariants()
    assert m.capacity().free_blocks == (4, 24 - 3)                       # positions 6..10 of the window: pages 3, 4, 5
    m.release("r")
    assert m.capacity().free_blocks == (6, 24)
    with pytest.raises(ValueError, match="page sizes"):
        manager([Need(0, KVCacheNeed(1, 16, block_size=0))])


def test_the_most_pages_a_request_holds_follow_the_window_of_each_group():
    """What admission compares with the pools: all pages where all keys are kept, the
    window's span (and the step's tokens) where a window has passed; measured here on
    a real run of the manager."""

    needs = [Need(0, KVCacheNeed(1, 16)), Need(1, KVCacheNeed(1, 16, window=6))]
    m = manager(needs, block_size=4, num_blocks=[64, 64], max_len=256)
    capacity = m.capacity()
    assert capacity.windows == (None, 6)
    assert capacity.most_pages_held(200, 200) == (50, 50)          # one step brings everything
    assert capacity.most_pages_held(200, 1) == (50, 3)             # single tokens: 6 keys over at most 3 pages
    assert capacity.most_pages_held(200, 7) == (50, 4)
    assert capacity.most_pages_held(3, 7) == (1, 1)
    for step_tokens in (1, 3, 7, 16):
        m.admit("r")
        length, most = 0, 0
        while length < 120:
            step = m.prepare_step([StepItem("r", length, length + step_tokens)])
            most = max(most, 64 - m.capacity().free_blocks[1])
            m.commit_step(step)
            length += step_tokens
        assert most <= capacity.most_pages_held(120, step_tokens)[1]
        assert most >= capacity.most_pages_held(120, step_tokens)[1] - 1        # the bound is not loose
        m.release("r")


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page(seed):
    """Requests arrive, grow by portions, abort, end, in random order: after every
    operation no page is lost, held twice or freed twice."""

    rng = random.Random(seed)
    needs = [Need(0, KVCacheNeed(1, 8)), Need(1, KVCacheNeed(1, 8, window=5)), Need(2, StateNeed((3,)))]
    m = manager(needs, block_size=4, num_blocks=[12, 6], slots=3, max_len=40)
    lengths: dict[str, int] = {}
    counter = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.2 and len(lengths) < 3:
            name = f"r{counter}"
            counter += 1
            m.admit(name)
            lengths[name] = 0
        elif action < 0.3 and lengths:
            name = rng.choice(sorted(lengths))
            m.release(name)
            del lengths[name]
        elif lengths:
            chosen = [n for n in sorted(lengths) if rng.random() < 0.7 and lengths[n] < 40]
            items = [StepItem(n, lengths[n], min(40, lengths[n] + rng.choice((1, 1, 2, 5, 9)))) for n in chosen]
            if not items:
                continue
            try:
                step = m.prepare_step(items)
            except OutOfPagesError:
                m.assert_invariants()
                continue
            m.assert_invariants()
            if rng.random() < 0.25:
                m.abort_step(step)
            else:
                m.commit_step(step)
                for item in items:
                    lengths[item.request_id] = item.end
        m.assert_invariants()
        for name, length in lengths.items():
            assert m.committed_tokens(name) == length
    for name in list(lengths):
        m.release(name)
    m.assert_invariants()
    assert m.capacity().free_blocks == (12, 6) and m.capacity().free_slots == 3


def test_a_spare_page_and_a_spare_state_slot_that_no_request_gets():
    """Storage has one page and one state slot more than the manager hands out."""

    import torch

    made = manager([Need(0, KVCacheNeed(2, 4)), Need(1, StateNeed((3,)))], block_size=4, num_blocks=5, slots=2, max_len=20)
    made.allocate_storage(torch.float32, "cpu")
    assert made.key_pools[0].shape[1] == 6 and made.value_pools[0].shape[1] == 6
    assert made.state_tensors[0].shape == (3, 3)
    assert made.spare_page(0) == 5 and made.spare_state_slot == 2
    assert {made.admit("a"), made.admit("b")} == {0, 1}
    made.commit_step(made.prepare_step([StepItem("a", 0, 12), StepItem("b", 0, 8)]))
    pages = set(made.block_table("a")) | set(made.block_table("b"))
    assert pages == {0, 1, 2, 3, 4} and made.capacity().free_blocks == (0,)
