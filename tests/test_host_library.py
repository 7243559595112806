"""The host library's C ABI, called directly (no GPU): what the Python faces rely on."""

import ctypes

import numpy as np

from flyweight_amd import host


def test_the_library_builds_loads_and_names_its_abi():
    lib = host.library()
    assert lib.fwh_abi_version() == host.ABI_VERSION


def test_pool_codes():
    lib = host.library()
    pool = lib.fwh_pool_create(3)
    try:
        assert [lib.fwh_pool_alloc(pool) for _ in range(3)] == [0, 1, 2]
        assert lib.fwh_pool_alloc(pool) == host.OUT_OF_PAGES and "out of" in host.last_error()
        assert lib.fwh_pool_free(pool, 1) == 0 and lib.fwh_pool_free(pool, 1) == host.ERROR
        assert "not held" in host.last_error()
        assert lib.fwh_pool_alloc(pool) == 1 and lib.fwh_pool_peak(pool) == 3 and lib.fwh_pool_free_count(pool) == 0
    finally:
        lib.fwh_pool_destroy(pool)
    assert not lib.fwh_pool_create(0) and "at least one" in host.last_error()


def test_cache_reservations_are_all_or_nothing_and_windows_give_pages_back():
    lib = host.library()
    windows = (ctypes.c_int * 2)(0, 100)            # every key; the last 100 keys
    cache = lib.fwh_cache_create(2, windows, 6, 2, 64, 0)
    try:
        assert lib.fwh_cache_admit(cache, 7) == 0 and lib.fwh_cache_admit(cache, 7) == host.ERROR
        assert lib.fwh_cache_reserve(cache, 7, 64 * 7) == host.OUT_OF_PAGES         # 7 pages of 6
        missing = host.ints(2)
        lib.fwh_cache_pages_missing(cache, 7, 200, missing)
        assert list(missing[:2]) == [4, 4]                                          # nothing was taken
        assert lib.fwh_cache_reserve(cache, 7, 300) == 0 and lib.fwh_cache_commit(cache, 7, 300) == 0
        pages = host.ints(8)
        assert lib.fwh_cache_table(cache, 7, 0, pages, 8) == 5 and list(pages[:5]) == [0, 1, 2, 3, 4]
        # the window of 100 starts at key 201: blocks 0..2 were given back
        assert lib.fwh_cache_table(cache, 7, 1, pages, 8) == 5 and list(pages[:5]) == [-1, -1, -1, 3, 4]
        rows = np.full((1, 6), 9, dtype=np.int32)
        assert lib.fwh_cache_fill_tables(cache, 1, (ctypes.c_int64 * 1)(7), 1, 6, rows.ctypes.data) == 0
        assert rows.tolist() == [[0, 0, 0, 3, 4, 0]]
        assert lib.fwh_cache_fill_tables(cache, 1, (ctypes.c_int64 * 1)(7), 1, 4, rows.ctypes.data) == host.ERROR
        assert lib.fwh_cache_commit(cache, 7, 10) == host.ERROR and "shrink" in host.last_error()
        assert lib.fwh_cache_check(cache) == 0
        assert lib.fwh_cache_release(cache, 7) == 0 and lib.fwh_cache_release(cache, 7) == host.ERROR
        assert lib.fwh_pool_free_count(lib.fwh_cache_group_pool(cache, 1)) == 6
    finally:
        lib.fwh_cache_destroy(cache)


def test_scheduler_through_the_c_entry_points():
    lib = host.library()
    windows = (ctypes.c_int * 1)(0)
    cache = lib.fwh_cache_create(1, windows, 8, 2, 64, 0)
    scheduler = lib.fwh_scheduler_create(cache, 512, 96, 64, 0, 2, 100)
    try:
        prompt = (ctypes.c_int * 70)(*range(70))
        none = (ctypes.c_int * 1)()
        assert lib.fwh_scheduler_submit(scheduler, prompt, 0, 4, none, 0) == host.ERROR and "empty" in host.last_error()
        assert lib.fwh_scheduler_submit(scheduler, prompt, 70, 500, none, 0) == host.ERROR and "context" in host.last_error()
        prompt[3] = 100     # the vocabulary given above has 100 entries
        assert lib.fwh_scheduler_submit(scheduler, prompt, 70, 2, none, 0) == host.ERROR and "place 3" in host.last_error()
        prompt[3] = 3
        assert lib.fwh_scheduler_submit(scheduler, prompt, 70, 2, (ctypes.c_int * 1)(-1), 1) == host.ERROR and "stop token" in host.last_error()
        first = lib.fwh_scheduler_submit(scheduler, prompt, 70, 2, none, 0)
        second = lib.fwh_scheduler_submit(scheduler, prompt, 40, 2, (ctypes.c_int * 1)(5), 1)
        assert (first, second) == (1, 2)
        assert lib.fwh_scheduler_submit(scheduler, prompt, 3, 1, none, 0) == host.ERROR and "queue" in host.last_error()
        counts = host.ints(7)
        assert lib.fwh_scheduler_schedule(scheduler, counts) == 0
        assert list(counts) == [2, 96, 0, 0, 2, 0, 64]  # a portion of 64, then 32 of the second prompt: the budget; a page each
        owners, lengths, wants, tokens = host.ids(2), host.ints(2), host.ints(2), host.ints(96)
        lib.fwh_plan_segments(scheduler, owners, lengths, wants, tokens)
        assert list(owners) == [1, 2] and list(lengths) == [64, 32] and list(wants) == [0, 0]
        assert list(tokens[:64]) == list(range(64)) and list(tokens[64:96]) == list(range(32))
        ev_owner, ev_value, ev_kind = host.ids(8), host.ints(8), host.ints(8)
        n = lib.fwh_scheduler_complete(scheduler, host.ids(0), host.ints(0), 0, ev_owner, ev_value, ev_kind, 8)
        assert [(ev_owner[i], ev_value[i], ev_kind[i]) for i in range(n)] == [(1, 64, 3), (2, 32, 3)]
        assert lib.fwh_scheduler_schedule(scheduler, counts) == 0 and list(counts)[:2] == [2, 14]
        lib.fwh_plan_segments(scheduler, owners, lengths, wants, tokens)
        assert list(lengths) == [6, 8] and list(wants) == [1, 1]
        # a plan whose wanted tokens are not handed over is refused, and nothing has changed
        assert lib.fwh_scheduler_complete(scheduler, host.ids(0), host.ints(0), 0, ev_owner, ev_value, ev_kind, 8) == host.ERROR
        info = host.ints(9)
        assert lib.fwh_request_info(scheduler, 1, info) == 0 and info[0] == 64
        drawn = (ctypes.c_int * 2)(9, 5)
        n = lib.fwh_scheduler_complete(scheduler, (ctypes.c_int64 * 2)(1, 2), drawn, 2, ev_owner, ev_value, ev_kind, 8)
        # the second request drew its stop token: it is finished and its pages are back
        assert [(ev_owner[i], ev_value[i], ev_kind[i]) for i in range(n)] == [(1, 9, 0), (2, 5, 0), (2, 1, 1)]
        assert lib.fwh_cache_is_live(cache, 2) == 0 and lib.fwh_cache_is_live(cache, 1) == 1
    finally:
        lib.fwh_scheduler_destroy(scheduler)
        lib.fwh_cache_destroy(cache)
