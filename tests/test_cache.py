"""The cache manager on the host: no page lost, held twice or freed twice, under
random orders of requests; all-or-nothing reservations; windows give pages back;
state slots.  Vectors follow the reference's tests/test_alloc.py."""

import random

import pytest

from paged_attention_engine_amd.cache import (HOLE, AllocStatus, BlockAllocator, CacheManager, PagedSpec, attention_pages,
                                              StateSpec)


def check_allocator(alloc: BlockAllocator):
    """tests/test_alloc.py:44-65: every page is in exactly one place."""
    free = list(alloc.free_block_ids())
    held = []
    for seq in alloc.sequence_ids():
        table = alloc.block_table(seq)
        live = [b for b in table if b != HOLE]
        held += live
        assert len(table) == alloc.blocks_needed(alloc.num_tokens(seq))
        assert alloc.blocks_held(seq) == len(live)
    assert len(free) == len(set(free)) and len(held) == len(set(held))
    assert not set(free) & set(held)
    assert sorted(free + held) == list(range(alloc.num_blocks))
    assert alloc.num_free + alloc.num_allocated == alloc.num_blocks
    alloc.audit()  # the allocator's own check of the same, page by page


def test_allocator_invariants_under_random_operations():
    rng = random.Random(0)
    alloc = BlockAllocator(24, 4)
    live, next_id, exhausted = [], 0, 0
    for _ in range(4000):  # tests/test_alloc.py:85-140
        op = rng.random()
        if op < 0.25 or not live:
            alloc.create_sequence(next_id)
            live.append(next_id)
            next_id += 1
        elif op < 0.8:
            seq = rng.choice(live)
            before = (alloc.free_block_ids(), {s: (alloc.block_table(s), alloc.num_tokens(s)) for s in live})
            result = alloc.append_tokens(seq, rng.randint(1, 9))
            if not result.ok:
                exhausted += 1
                after = (alloc.free_block_ids(), {s: (alloc.block_table(s), alloc.num_tokens(s)) for s in live})
                assert before == after  # a failed allocation touches nothing
        elif op < 0.9:
            seq = rng.choice(live)
            alloc.release_before(seq, rng.randint(0, alloc.num_tokens(seq) + 3))
        else:
            seq = live.pop(rng.randrange(len(live)))
            alloc.free_sequence(seq)
        check_allocator(alloc)
    assert exhausted > 0
    for seq in live:
        alloc.free_sequence(seq)
    check_allocator(alloc)
    assert alloc.num_free == 24


def test_allocation_is_all_or_nothing_and_fifo():
    alloc = BlockAllocator(4, 4)
    alloc.create_sequence(0)
    assert alloc.append_tokens(0, 9).new_block_ids == (0, 1, 2)
    alloc.create_sequence(1)
    assert alloc.append_tokens(1, 5).status is AllocStatus.OUT_OF_BLOCKS  # needs 2, 1 free
    assert alloc.num_tokens(1) == 0 and alloc.block_table(1) == () and alloc.num_free == 1
    assert alloc.append_tokens(1, 4).new_block_ids == (3,)
    assert alloc.free_sequence(0) == (0, 1, 2)
    # freed pages go to the rear: reuse is as late as possible (engine/cache.py:180-184)
    assert alloc.free_block_ids() == (0, 1, 2)
    alloc.free_sequence(1)
    assert alloc.free_block_ids() == (0, 1, 2, 3)


def test_a_page_is_taken_exactly_on_the_token_that_overflows():
    alloc = BlockAllocator(8, 4)  # tests/test_alloc.py:215-228
    alloc.create_sequence(7)
    taken = [len(alloc.append_token(7).new_block_ids) for _ in range(9)]
    assert taken == [1, 0, 0, 0, 1, 0, 0, 0, 1]
    assert alloc.physical_slot(7, 5) == (alloc.block_table(7)[1], 1)
    with pytest.raises(IndexError):
        alloc.physical_slot(7, 9)


def test_caller_bugs_raise():
    alloc = BlockAllocator(2, 4)
    alloc.create_sequence(1)
    with pytest.raises(KeyError):
        alloc.create_sequence(1)
    with pytest.raises(KeyError):
        alloc.append_tokens(2, 1)
    alloc.free_sequence(1)
    with pytest.raises(KeyError):
        alloc.free_sequence(1)  # double free
    with pytest.raises(ValueError):
        BlockAllocator(0, 4)


def test_window_pages_come_back_and_leave_holes():
    alloc = BlockAllocator(8, 4)
    alloc.create_sequence(0)
    alloc.append_tokens(0, 14)  # logical blocks 0..3
    assert alloc.release_before(0, 9) == (0, 1)  # positions 0..7 lie wholly before 9
    assert alloc.block_table(0) == (HOLE, HOLE, 2, 3)
    assert alloc.release_before(0, 9) == ()  # nothing is given back twice
    with pytest.raises(IndexError):
        alloc.physical_slot(0, 3)
    assert alloc.physical_slot(0, 9) == (2, 1)
    alloc.append_tokens(0, 6)  # grows past the holes
    assert len(alloc.block_table(0)) == 5
    assert alloc.free_sequence(0) == (2, 3, 4)
    check_allocator(alloc)


def two_group_manager(num_blocks=6, slots=3):
    paged = [attention_pages(2, 16), attention_pages(2, 16), attention_pages(2, 16, window=6), attention_pages(2, 16, window=6), None]
    states = [None, None, None, None, StateSpec((4,))]
    return CacheManager(paged, states, block_size=4, num_blocks=num_blocks, num_slots=slots, device=None)


def test_groups_are_formed_by_need():
    cache = two_group_manager()
    assert len(cache.groups) == 2
    assert cache.groups[0].entries == [0, 1] and cache.groups[1].entries == [2, 3]
    assert cache.group_of(3) == 1 and cache.group_of(4) is None


def test_reservation_spans_all_groups_or_none():
    cache = two_group_manager(num_blocks={None: 3, 6: 6})
    assert cache.create_sequence(0) and cache.create_sequence(1)
    assert cache.reserve(0, 8).ok  # two pages in each group
    before = cache.free_blocks()
    assert not cache.reserve(1, 8).ok  # the full group has one page left
    assert cache.free_blocks() == before and cache.num_tokens(1) == 0
    assert cache.block_table(1, 1) == ()  # nothing was taken in the windowed group either
    assert cache.reserve(1, 4).ok


def test_release_passed_follows_the_window():
    cache = two_group_manager(num_blocks=8)
    cache.create_sequence(0)
    cache.reserve(0, 13)
    # next query stands at 13 and sees keys from 13 - 6 + 1 = 8: pages of positions 0..7 go
    assert cache.release_passed(0) == 2
    assert cache.block_table(1, 0)[:2] == (HOLE, HOLE) and HOLE not in cache.block_table(0, 0)
    assert cache.release_passed(0) == 0
    assert cache.free_sequence(0) == 4 + 2
    assert cache.free_blocks() == (8, 8)


def test_capacity_arithmetic_accounts_for_windows():
    cache = two_group_manager(num_blocks={None: 10, 6: 4})
    # windowed group: window - 1 + chunk = 9 tokens span at most ceil(9 / 4) + 1 = 4 pages
    assert cache.groups[1].max_blocks_for(36, 4) == 4
    assert cache.fits_alone(36, margin=0, max_chunk=4)
    assert not cache.fits_alone(36, margin=1, max_chunk=4)
    assert not cache.fits_alone(36, margin=1, max_chunk=None)  # a whole 36-token step needs 9 windowed pages
    assert not cache.fits_alone(44, margin=0, max_chunk=4)     # 11 pages in the full group


def test_state_slots():
    cache = two_group_manager(slots=2)
    assert cache.create_sequence(10) and cache.create_sequence(11)
    assert {cache.slot_of(10), cache.slot_of(11)} == {0, 1}
    assert not cache.create_sequence(12)  # no slot: nothing registered
    assert not cache.has_sequence(12)
    cache.free_sequence(10)
    assert cache.create_sequence(12) and cache.slot_of(12) == 0
    with pytest.raises(KeyError):
        cache.create_sequence(12)


def test_manager_under_random_requests():
    rng = random.Random(3)
    cache = two_group_manager(num_blocks={None: 12, 6: 7}, slots=4)
    live, next_id = [], 0
    for _ in range(3000):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            assert cache.create_sequence(next_id)
            live.append(next_id)
            next_id += 1
        elif op < 0.8 and live:
            seq = rng.choice(live)
            n = rng.randint(1, 7)
            expect = cache.can_reserve(seq, n)
            tokens = cache.num_tokens(seq)
            assert cache.reserve(seq, n).ok == expect
            assert cache.num_tokens(seq) == tokens + (n if expect else 0)
            cache.release_passed(seq)
        elif live:
            cache.free_sequence(live.pop(rng.randrange(len(live))))
        for group in cache.groups:
            check_allocator(group.allocator)
            assert set(group.allocator.sequence_ids()) == set(live)
        assert sorted(cache.slots.held()) == sorted(live)
        assert cache.slots.num_free + len(live) == 4
    for seq in live:
        cache.free_sequence(seq)
    assert cache.free_blocks() == (12, 7)


def test_a_page_cannot_come_back_twice_or_from_a_stranger():
    alloc = BlockAllocator(4, 4)
    alloc.create_sequence(0)
    alloc.create_sequence(1)
    alloc.append_tokens(0, 8)
    alloc.append_tokens(1, 4)
    page = alloc.block_table(1)[0]
    with pytest.raises(AssertionError):
        alloc._give_back(0, page)  # sequence 0 does not hold it
    alloc.free_sequence(1)
    with pytest.raises(AssertionError):
        alloc._give_back(1, page)  # it is free already
    alloc.audit()
    assert alloc.num_free == 2 and alloc.free_block_ids() == (3, page)


def test_the_table_array_is_the_table():
    alloc = BlockAllocator(6, 2)
    alloc.create_sequence(3)
    alloc.append_tokens(3, 5)
    view = alloc.table_array(3)
    assert list(view) == list(alloc.block_table(3)) == [0, 1, 2]
    alloc.release_before(3, 2)
    assert list(view) == [HOLE, 1, 2]  # not a copy: the step's staging buffer reads the live table


def test_pages_hold_what_the_mixer_declares():
    from paged_attention_engine_amd.cache import PAGE, PagedTensor, bytes_of_one_page_everywhere
    import torch

    latent = PagedSpec((PagedTensor("latent", (PAGE, 24)),))
    kv = attention_pages(2, 16, window=6)
    assert kv.elements_per_token() == 2 * 2 * 16 and latent.elements_per_token() == 24
    assert [t.shape(4) for t in kv.tensors] == [(2, 4, 16), (2, 16, 4)]
    # stops 0 and 1 share a group (same spec), stop 2 has its own; the byte arithmetic counts every stop
    assert bytes_of_one_page_everywhere([kv, kv, latent, None], 4, torch.bfloat16) == (2 * 64 + 24) * 4 * 2
    cache = CacheManager([kv, kv, latent, None], [None] * 4, block_size=4, num_blocks=5, num_slots=2, device=None)
    assert [g.entries for g in cache.groups] == [[0, 1], [2]]
    assert cache.storage_bytes() == 5 * (2 * 64 + 24) * 4 * 4  # float32 by default
    assert cache.padding_page(0) == 5 and cache.padding_slot == 2
    with pytest.raises(ValueError):
        PagedTensor("x", (3, 4))           # no PAGE axis
    with pytest.raises(ValueError):
        PagedSpec((PagedTensor("a", (PAGE,)), PagedTensor("a", (PAGE, 2))))  # one name twice
