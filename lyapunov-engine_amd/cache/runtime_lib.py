"""Loads the host runtime library (cache manager and scheduler, C++) and
declares its C interface for ctypes."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_void_p

from ..kernels import build

_lib = None


class RuntimeError_(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    try:
        L = ctypes.CDLL(str(build.runtime_library()))
    except OSError as e:
        raise RuntimeError_(f"cannot load the host runtime library: {e}") from None
    i32p, i64p = POINTER(c_int32), POINTER(c_int64)
    L.lyp_rt_last_error.restype = c_char_p
    L.lyp_cache_create.restype = c_void_p
    L.lyp_cache_create.argtypes = [c_int, POINTER(c_int), POINTER(c_int), POINTER(c_int), c_int]
    L.lyp_cache_destroy.argtypes = [c_void_p]
    for name in ("add", "has", "length", "capacity", "free", "state_slot", "max_length"):
        getattr(L, f"lyp_cache_{name}").argtypes = [c_void_p, c_int64]
    for name in ("can_extend", "extend", "commit"):
        getattr(L, f"lyp_cache_{name}").argtypes = [c_void_p, c_int64, c_int]
    L.lyp_cache_reset.argtypes = [c_void_p]
    L.lyp_cache_num_free_pages.argtypes = [c_void_p, c_int]
    L.lyp_cache_num_free_slots.argtypes = [c_void_p]
    L.lyp_cache_num_requests.argtypes = [c_void_p]
    L.lyp_cache_table.argtypes = [c_void_p, c_int64, c_int, i32p, c_int]
    L.lyp_cache_export.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]
    L.lyp_cache_reserve.argtypes = [c_void_p, c_void_p, c_void_p, c_int]
    L.lyp_cache_step_tables.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p,
                                        c_void_p]
    L.lyp_cache_ref_count.argtypes = [c_void_p, c_int, c_int]
    L.lyp_cache_check.argtypes = [c_void_p]
    L.lyp_cache_counters.argtypes = [c_void_p, i64p]
    L.lyp_cache_counters.restype = None

    L.lyp_sched_create.restype = c_void_p
    L.lyp_sched_create.argtypes = [c_void_p, c_int, c_int, c_int, c_int, i32p, c_int]
    L.lyp_sched_destroy.argtypes = [c_void_p]
    L.lyp_sched_add.argtypes = [c_void_p, c_int64, i32p, c_int, c_int, c_int]
    L.lyp_sched_abort.argtypes = [c_void_p, c_int64]
    for name in ("has_unfinished", "num_waiting", "num_running"):
        getattr(L, f"lyp_sched_{name}").argtypes = [c_void_p]
    L.lyp_sched_schedule.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int]
    L.lyp_sched_post_step.argtypes = [c_void_p, i32p, c_int]
    L.lyp_sched_post_step_status.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int]
    L.lyp_sched_plan_tokens.argtypes = [c_void_p, c_void_p, c_int]
    L.lyp_sched_last_preempted.argtypes = [c_void_p, i64p, c_int]
    L.lyp_sched_info.argtypes = [c_void_p, c_int64, i32p]
    L.lyp_sched_tokens.argtypes = [c_void_p, c_int64, c_int, i32p, c_int]
    L.lyp_sched_forget.argtypes = [c_void_p, c_int64]
    L.lyp_sched_counters.argtypes = [c_void_p, i64p]
    L.lyp_sched_counters.restype = None
    _lib = L
    return L


def last_error() -> str:
    return lib().lyp_rt_last_error().decode()
