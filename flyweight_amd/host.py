"""The host library (``csrc/host``: cache bookkeeping and scheduler in C++ behind a flat C ABI),
loaded with ctypes. ``library()`` builds it at its first call if nothing current is built."""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int64, c_void_p
from typing import Optional

from .kernels.build import ensure_host_built

ERROR, OUT_OF_PAGES, NO_PAGE = -1, -2, -1
NOT_DECODE_ONLY = -3
ABI_VERSION = 5

_LIB: Optional[ctypes.CDLL] = None
_INTS, _IDS = POINTER(c_int), POINTER(c_int64)

_SIGNATURES = {
    "fwh_last_error": (c_char_p, []),
    "fwh_abi_version": (c_int, []),
    "fwh_pool_create": (c_void_p, [c_int]),
    "fwh_pool_destroy": (None, [c_void_p]),
    "fwh_pool_alloc": (c_int, [c_void_p]),
    "fwh_pool_free": (c_int, [c_void_p, c_int]),
    "fwh_pool_size": (c_int, [c_void_p]),
    "fwh_pool_free_count": (c_int, [c_void_p]),
    "fwh_pool_peak": (c_int, [c_void_p]),
    "fwh_pool_is_held": (c_int, [c_void_p, c_int]),
    "fwh_cache_create": (c_void_p, [c_int, _INTS, c_int, c_int, c_int, c_int]),
    "fwh_cache_create_sized": (c_void_p, [c_int, _INTS, _INTS, c_int, c_int, c_int]),
    "fwh_cache_destroy": (None, [c_void_p]),
    "fwh_cache_group_pool": (c_void_p, [c_void_p, c_int]),
    "fwh_cache_slot_pool": (c_void_p, [c_void_p]),
    "fwh_cache_admit": (c_int, [c_void_p, c_int64]),
    "fwh_cache_reserve": (c_int, [c_void_p, c_int64, c_int]),
    "fwh_cache_commit": (c_int, [c_void_p, c_int64, c_int]),
    "fwh_cache_truncate": (c_int, [c_void_p, c_int64, c_int]),
    "fwh_cache_truncate_batch": (c_int, [c_void_p, _IDS, _INTS, c_int]),
    "fwh_cache_release": (c_int, [c_void_p, c_int64]),
    "fwh_cache_is_live": (c_int, [c_void_p, c_int64]),
    "fwh_cache_slot_of": (c_int, [c_void_p, c_int64]),
    "fwh_cache_length_of": (c_int, [c_void_p, c_int64]),
    "fwh_cache_pages_missing": (c_int, [c_void_p, c_int64, c_int, _INTS]),
    "fwh_cache_table": (c_int, [c_void_p, c_int64, c_int, _INTS, c_int]),
    "fwh_cache_fill_tables": (c_int, [c_void_p, c_int, _IDS, c_int, c_int, c_void_p]),
    "fwh_cache_longest_table": (c_int, [c_void_p, c_int, _IDS, c_int]),
    "fwh_cache_describe": (c_int, [c_void_p, _IDS, c_int, _INTS, _INTS]),
    "fwh_cache_reserve_batch": (c_int, [c_void_p, _IDS, _INTS, c_int]),
    "fwh_cache_commit_batch": (c_int, [c_void_p, _IDS, _INTS, c_int]),
    "fwh_cache_live": (c_int, [c_void_p, _IDS, c_int]),
    "fwh_cache_check": (c_int, [c_void_p]),
    "fwh_scheduler_create": (c_void_p, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int]),
    "fwh_scheduler_destroy": (None, [c_void_p]),
    "fwh_scheduler_submit": (c_int64, [c_void_p, _INTS, c_int, c_int, _INTS, c_int]),
    "fwh_scheduler_cancel": (c_int, [c_void_p, c_int64]),
    "fwh_scheduler_fail": (c_int, [c_void_p, c_int64, c_char_p]),
    "fwh_scheduler_has_work": (c_int, [c_void_p]),
    "fwh_scheduler_preemptions": (c_int, [c_void_p]),
    "fwh_scheduler_queue": (c_int, [c_void_p, c_int, _IDS, c_int]),
    "fwh_scheduler_schedule": (c_int, [c_void_p, _INTS]),
    "fwh_plan_segments": (c_int, [c_void_p, _IDS, _INTS, _INTS, _INTS]),
    "fwh_plan_list": (c_int, [c_void_p, c_int, _IDS]),
    "fwh_scheduler_complete": (c_int, [c_void_p, _IDS, _INTS, c_int, _IDS, _INTS, _INTS, c_int]),
    "fwh_plan_fill_decode": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int]),
    "fwh_scheduler_complete_ordered": (c_int, [c_void_p, _INTS, c_int, _IDS, _INTS, _INTS, c_int]),
    "fwh_plan_steps_ahead": (c_int, [c_void_p, c_int, _IDS, c_int]),
    "fwh_plan_budgets": (c_int, [c_void_p, _INTS, c_int]),
    "fwh_request_info": (c_int, [c_void_p, c_int64, _INTS]),
    "fwh_request_generated": (c_int, [c_void_p, c_int64, _INTS, c_int]),
    "fwh_request_error": (c_char_p, [c_void_p, c_int64]),
    "fwh_scheduler_hold_admissions": (c_int, [c_void_p, c_int]),
    "fwh_scheduler_forget": (c_int, [c_void_p, c_int64]),
}


def library() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        lib = ctypes.CDLL(ensure_host_built())
        for name, (restype, argtypes) in _SIGNATURES.items():
            entry = getattr(lib, name)
            entry.restype, entry.argtypes = restype, argtypes
        if lib.fwh_abi_version() != ABI_VERSION:
            raise RuntimeError(f"the host library has ABI {lib.fwh_abi_version()}, this package expects {ABI_VERSION}")
        _LIB = lib
    return _LIB


def last_error() -> str:
    return library().fwh_last_error().decode("utf-8", "replace")


def ints(count: int):
    return (c_int * max(count, 1))()


def ids(count: int):
    return (c_int64 * max(count, 1))()
