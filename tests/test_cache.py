"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice."""

import random

import pytest
import torch

from flyweight_amd.cache import (CacheAccountingError, CacheManager, CacheNeed, FixedState, NO_PAGE, OutOfPages, PagedKV,
                                 PagePool, SlotPool)

KV = PagedKV(num_kv_heads=2, head_dim=16)
NEEDS = {0: FixedState((8, 2)), 1: KV, 2: FixedState((8, 2)), 3: KV}


def test_pool_is_lifo_and_refuses_double_free():
    pool = PagePool(4)
    a, b = pool.alloc(), pool.alloc()
    assert (a, b) == (0, 1) and pool.in_use == 2
    pool.free(a)
    assert pool.alloc() == a            # the page given back is the next one handed out
    pool.free(b)
    with pytest.raises(CacheAccountingError):
        pool.free(b)
    with pytest.raises(CacheAccountingError):
        pool.free(3)                    # never handed out
    for _ in range(pool.free_count):
        pool.alloc()
    with pytest.raises(OutOfPages):
        pool.alloc()
    slots = SlotPool(2)
    s = slots.alloc()
    slots.free(s)
    with pytest.raises(CacheAccountingError):
        slots.free(s)


def test_lifecycle_of_the_reference_contract():
    # native/tests/paged_kv_contract.cpp:244-296: 64 pages; 100 tokens -> 2 pages, 200 -> 4, release -> none
    cache = CacheManager({0: KV}, num_pages=64, max_requests=2)
    cache.admit("r")
    cache.reserve("r", 100)
    assert cache.groups[0].pool.in_use == 2
    cache.reserve("r", 200)
    assert cache.groups[0].pool.in_use == 4
    cache.reserve("r", 150)             # never shrinks a mapping
    assert cache.groups[0].pool.in_use == 4
    cache.commit("r", 200)
    cache.release("r")
    assert cache.groups[0].pool.in_use == 0 and cache.groups[0].pool.free_count == 64
    cache.check_invariants()


def test_truncate_of_the_reference_contract():
    # native/tests/paged_kv_contract.cpp:244-296: 64 pages; one sequence of 100 tokens (2 pages), one
    # of 200 (4); the second cut back to 128 tokens keeps exactly 2 pages; releases leave none out
    cache = CacheManager({0: KV}, num_pages=64, max_requests=2)
    pool = cache.groups[0].pool
    cache.admit("one")
    cache.admit("two")
    cache.reserve("one", 100)
    assert len(cache.groups[0].tables["one"]) == 2 and pool.free_count == 62
    cache.reserve("two", 200)
    cache.commit("two", 200)
    assert len(cache.groups[0].tables["two"]) == 4 and pool.free_count == 58
    kept = cache.groups[0].tables["two"][:2]
    cache.truncate("two", 128)
    assert cache.groups[0].tables["two"] == kept and pool.free_count == 60 and cache.length_of("two") == 128
    cache.check_invariants()
    cache.truncate("two", 129)          # one token more would need a third page: nothing to give back
    assert len(cache.groups[0].tables["two"]) == 2
    cache.release("one")
    assert pool.free_count == 62
    cache.release("two")
    assert pool.free_count == 64
    cache.check_invariants()


def test_truncate_drops_reservations_but_never_rewinds_state_or_a_window():
    cache = CacheManager(NEEDS, num_pages=6, max_requests=3)
    cache.admit("r")
    cache.reserve("r", 70)
    cache.commit("r", 70)
    cache.reserve("r", 200)             # a step that will not run after all
    assert cache.groups[0].pool.in_use == 4
    cache.drop_reservations(["r"])
    assert cache.groups[0].pool.in_use == 2 and cache.length_of("r") == 70
    with pytest.raises(CacheAccountingError, match="fixed-size state"):
        cache.truncate("r", 10)         # the state slot has seen 70 tokens and cannot go back
    cache.check_invariants()
    windowed = CacheManager({0: PagedKV(1, 16, window=70)}, num_pages=8, max_requests=1)
    windowed.admit("w")
    windowed.reserve("w", 300)
    windowed.commit("w", 300)           # keys before 231 are gone: blocks 0..2 were given back
    assert windowed.groups[0].tables["w"][:3] == [-1, -1, -1]
    windowed.truncate("w", 280)         # needs keys from 211 on: block 3 onwards, all there
    assert windowed.length_of("w") == 280
    with pytest.raises(CacheAccountingError, match="window has passed"):
        windowed.truncate("w", 200)     # would need keys from 131 on: block 2 is gone
    windowed.check_invariants()
    windowed.release("w")
    assert windowed.groups[0].pool.free_count == 8


def test_groups_share_pages_across_their_layers_and_slots_across_states():
    cache = CacheManager(NEEDS, num_pages=6, max_requests=3, device=torch.device("cpu"))
    assert len(cache.groups) == 1 and cache.groups[0].entries == [1, 3]
    assert cache.entry_group == {1: 0, 3: 0}
    assert set(cache.state) == {0, 2} and cache.state[0].shape == (3 + 1, 8, 2)      # one spare slot behind the pool's
    assert cache.k_pages[1].shape == (6 + 1, 2, 64, 16) and cache.v_pages[3].shape == (6 + 1, 2, 16, 64)
    other = CacheManager({0: KV, 1: PagedKV(2, 16, window=100), 2: PagedKV(4, 16)}, num_pages=4, max_requests=1)
    assert len(other.groups) == 3       # a window or another head count is a group of its own


def test_reservation_is_all_or_nothing():
    cache = CacheManager({0: KV, 1: PagedKV(1, 32)}, num_pages=3, max_requests=2)
    cache.admit("a")
    cache.admit("b")
    cache.reserve("a", 128)
    with pytest.raises(OutOfPages):
        cache.reserve("b", 129)         # needs 3 pages, 1 free in both groups
    assert all(g.pool.in_use == 2 for g in cache.groups) and cache.groups[0].tables["b"] == []
    assert not cache.can_reserve("b", 129) and cache.can_reserve("b", 64)
    cache.check_invariants()


def test_state_slot_is_zeroed_when_handed_out():
    cache = CacheManager({0: FixedState((4, 2))}, num_pages=1, max_requests=2, device=torch.device("cpu"))
    slot = cache.admit("a")
    cache.state[0][slot] = 7.0
    cache.release("a")
    assert cache.admit("b") == slot     # LIFO: the same slot again
    assert float(cache.state[0][slot].abs().sum()) == 0.0


def test_entries_with_equal_state_start_a_slot_together_and_others_on_their_own():
    class Counted(FixedState):
        """A need of a mixer's own: starts at 2, says so entry by entry (the inherited way)."""
        def allocate_together(self, count, units, page_size, dtype, device):
            return CacheNeed.allocate_together(self, count, units, page_size, dtype, device)

        def initial_together(self, together, slot):
            CacheNeed.initial_together(self, together, slot)

        def initial(self, storage, slot):
            storage[slot] = 2.0

    needs = {0: FixedState((4, 2)), 1: FixedState((4, 2)), 2: FixedState((3,)), 5: FixedState((4, 2)), 7: Counted((4, 2)), 8: Counted((4, 2))}
    cache = CacheManager(needs, num_pages=1, max_requests=3, device=torch.device("cpu"))
    # the three equal entries lie in one tensor, the other shape and the other class apart
    assert cache.state[0].data_ptr() != cache.state[1].data_ptr()
    assert cache.state[0].untyped_storage().data_ptr() == cache.state[1].untyped_storage().data_ptr() == cache.state[5].untyped_storage().data_ptr()
    assert cache.state[2].untyped_storage().data_ptr() != cache.state[0].untyped_storage().data_ptr()
    assert cache.state[7].untyped_storage().data_ptr() != cache.state[8].untyped_storage().data_ptr()
    first, second = cache.admit("a"), cache.admit("b")
    for entry in needs:
        cache.state[entry][first] = 7.0
        cache.state[entry][second] = 9.0
    cache.release("a")
    assert cache.admit("c") == first
    for entry in needs:
        start = 2.0 if entry in (7, 8) else 0.0
        assert bool((cache.state[entry][first] == start).all()), entry
        assert bool((cache.state[entry][second] == 9.0).all()), entry       # the neighbour's slot is untouched


def test_window_group_gives_back_the_pages_its_window_has_passed():
    cache = CacheManager({0: PagedKV(1, 16, window=70), 1: PagedKV(1, 16)}, num_pages=8, max_requests=1)
    windowed, full = cache.groups
    cache.admit("r")
    cache.reserve("r", 300)
    cache.commit("r", 300)
    # the next query sits at 300 and sees keys 231..300: blocks 0..2 (tokens 0..191) are passed
    assert windowed.tables["r"][:3] == [NO_PAGE] * 3 and all(p != NO_PAGE for p in windowed.tables["r"][3:])
    assert windowed.pool.in_use == 2 and full.pool.in_use == 5
    cache.check_invariants()
    freed = windowed.pool.free_count
    cache.reserve("r", 330)             # one more block; a passed block is not mapped again
    assert windowed.pool.free_count == freed - 1
    cache.commit("r", 330)
    cache.release("r")
    assert windowed.pool.in_use == 0 and full.pool.in_use == 0
    rows = CacheManager({0: PagedKV(1, 16, window=70)}, num_pages=8, max_requests=1)
    rows.admit("r"); rows.reserve("r", 200); rows.commit("r", 200)
    table = rows.block_table_rows(0, ["r"])
    assert table.shape == (1, 4) and table.dtype.name == "int32" and (table >= 0).all()


def test_page_groups_are_sized_apart():
    """A group that keeps a window of keys beside one that keeps them all: each has a pool of its
    own size, a sequence is bounded by the group that keeps everything, and the windowed group
    serves it from a handful of pages that it keeps giving back."""
    window, full = PagedKV(1, 16, window=70), PagedKV(1, 16)
    cache = CacheManager({0: window, 1: full}, num_pages={window.group_key(): 3, full.group_key(): 10}, max_requests=2)
    windowed_group, full_group = cache.groups
    assert (windowed_group.pool.num_pages, full_group.pool.num_pages) == (3, 10)
    assert cache.num_pages == 10 and cache.group_pages == [3, 10] and cache.spare_pages == [3, 10]
    cache.admit("r")
    for length in range(60, 640, 60):       # portions of 60 tokens: the window never needs more than 3 pages at once
        cache.reserve("r", length)
        cache.commit("r", length)
        cache.check_invariants()
    assert full_group.pool.in_use == 10 and windowed_group.pool.in_use <= 3
    with pytest.raises(OutOfPages):
        cache.reserve("r", 641)             # the eleventh page of the group that keeps every key
    cache.release("r")
    assert windowed_group.pool.in_use == 0 and full_group.pool.in_use == 0
    # a portion that the windowed group cannot hold at once is refused whole: neither group changes
    cache.admit("s")
    with pytest.raises(OutOfPages):
        cache.reserve("s", 4 * 64)
    assert windowed_group.pool.in_use == 0 and full_group.pool.in_use == 0
    cache.check_invariants()
    # one number for the others, and names that match no group are refused
    other = CacheManager({0: window, 1: full}, num_pages={window.group_key(): 2, None: 7}, max_requests=1)
    assert other.group_pages == [2, 7]
    with pytest.raises(ValueError, match="do not exist"):
        CacheManager({0: full}, num_pages={window.group_key(): 2, None: 7}, max_requests=1)
    with pytest.raises(ValueError, match="no number of pages"):
        CacheManager({0: window, 1: full}, num_pages={window.group_key(): 2}, max_requests=1)


def test_misuse_is_refused():
    cache = CacheManager({0: KV}, num_pages=2, max_requests=1)
    cache.admit("a")
    with pytest.raises(CacheAccountingError):
        cache.admit("a")
    with pytest.raises(OutOfPages):
        cache.admit("b")                # no slot
    with pytest.raises(KeyError):
        cache.reserve("zz", 1)
    cache.release("a")
    with pytest.raises(CacheAccountingError):
        cache.release("a")
    small = CacheManager({0: KV}, num_pages=8, max_requests=1, max_pages_per_request=2)
    small.admit("a")
    with pytest.raises(OutOfPages, match="block table"):
        small.reserve("a", 129)


@pytest.mark.parametrize("seed", range(6))
def test_random_lifetimes_lose_nothing(seed):
    rng = random.Random(seed)
    cache = CacheManager({0: KV, 1: PagedKV(1, 32, window=100), 2: FixedState((4, 3))}, num_pages=12, max_requests=4)
    live = {}
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            cache.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.8 and live:
            request = rng.choice(list(live))
            grown = live[request] + rng.choice([1, 1, 1, 2, 7, 64, 130])
            try:
                cache.reserve(request, grown)
            except OutOfPages:
                victim = rng.choice(list(live))
                cache.release(victim)
                del live[victim]
            else:
                cache.commit(request, grown)
                live[request] = grown
        elif live:
            request = rng.choice(list(live))
            cache.release(request)
            del live[request]
        cache.check_invariants()
        assert set(cache.requests) == set(live)
    for request in list(live):
        cache.release(request)
    cache.check_invariants()
    assert all(g.pool.in_use == 0 for g in cache.groups) and cache.slots.free_count == 4
    assert max(g.pool.peak_in_use for g in cache.groups) > 6        # the pool was actually under pressure
