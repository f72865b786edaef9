"""Loads the host runtime library (cache manager, scheduler, step layout) and declares its C interface.

The library is plain C++ and is built on first use with the system's C++ compiler; it needs no GPU.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_long, c_void_p

from .csrc import build as _build

MISUSE, OUT_OF_PAGES, OUT_OF_SLOTS, SCHEDULER, STEP_REFUSED, INVALID, SAMPLER = -1, -2, -3, -4, -5, -6, -7

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None

H = c_void_p
PI = POINTER(c_int)
PI32 = POINTER(c_int32)
PI64 = POINTER(c_int64)
PL = POINTER(c_long)
PF = POINTER(c_float)
PD = POINTER(c_double)

_PROTOTYPES = {
    "leone_cache_create": (H, [PI, c_int, c_int, c_int]),
    "leone_cache_destroy": (None, [H]),
    "leone_cache_admit": (c_int, [H, c_int64]),
    "leone_cache_fork": (c_int, [H, c_int64, c_int64, c_int]),
    "leone_cache_truncate": (c_int, [H, c_int64, c_int]),
    "leone_cache_reserve": (c_int, [H, c_int64, c_int]),
    "leone_cache_commit": (c_int, [H, c_int64, c_int]),
    "leone_cache_rollback": (c_int, [H, c_int64]),
    "leone_cache_release": (c_int, [H, c_int64]),
    "leone_cache_has": (c_int, [H, c_int64]),
    "leone_cache_requests": (c_int, [H, PI64, c_int]),
    "leone_cache_length": (c_int, [H, c_int64]),
    "leone_cache_pending": (c_int, [H, c_int64]),
    "leone_cache_slot": (c_int, [H, c_int64]),
    "leone_cache_table": (c_int, [H, c_int64, c_int, PI, c_int]),
    "leone_cache_pages_needed": (c_int, [H, c_int64, c_int, PI]),
    "leone_cache_free_pages": (c_int, [H, c_int]),
    "leone_cache_free_list": (c_int, [H, c_int, PI, c_int]),
    "leone_cache_free_slots": (c_int, [H]),
    "leone_cache_free_slot_list": (c_int, [H, PI, c_int]),
    "leone_cache_holders": (c_int, [H, c_int, c_int]),
    "leone_cache_shared_pages": (c_int, [H, c_int]),
    "leone_cache_high_water": (c_int, [H, c_int]),
    "leone_cache_log_freed": (c_int, [H, c_int]),
    "leone_cache_drain_freed": (c_int, [H, c_int, PI, c_int]),
    "leone_cache_max_blocks": (c_int, [H, c_int]),
    "leone_cache_shortage": (None, [PI, PI, PI]),
    "leone_scheduler_create": (H, [H, PI64]),
    "leone_scheduler_destroy": (None, [H]),
    "leone_scheduler_submit": (c_int, [H, c_int64, PI32, c_int, c_int64, c_int]),
    "leone_scheduler_cancel": (c_int, [H, c_int64]),
    "leone_scheduler_has_work": (c_int, [H]),
    "leone_scheduler_plan": (c_int, [H]),
    "leone_scheduler_planned": (c_int, [H, PI64, PI, PI, PI, c_int]),
    "leone_scheduler_plan_ahead": (c_int, [H]),
    "leone_scheduler_ahead": (c_int, [H, PI64, PI, PI, PI, c_int]),
    "leone_scheduler_complete": (c_int, [H, PI64, PI32, c_int]),
    "leone_scheduler_abort": (c_int, [H]),
    "leone_scheduler_history": (c_int, [H, c_int64, PI32, c_int]),
    "leone_scheduler_tokens": (c_int, [H, c_int64, c_int, c_int, PI32]),
    "leone_scheduler_request_info": (c_int, [H, c_int64, PI, PI]),
    "leone_scheduler_live": (c_int, [H, PI64, c_int]),
    "leone_scheduler_queued": (c_int, [H, PI64, c_int]),
    "leone_scheduler_finished_count": (c_int, [H]),
    "leone_scheduler_finished_info": (c_int, [H, c_int, PI64, PI, PI, PI, PI]),
    "leone_scheduler_finished_tokens": (c_int, [H, c_int, PI32, PI32]),
    "leone_scheduler_event_count": (c_int, [H]),
    "leone_scheduler_events": (c_int, [H, c_int, c_int, PI, PI64, PI, PI, PI]),
    "leone_scheduler_stats": (None, [H, PI64]),
    "leone_sample_rows": (c_int, [PF, c_int, c_int, PD, PI, PI, PD, PD, PI]),
    "leone_step_pack": (c_long, [H, c_int, PI64, PI, PI, PI32, PI32, PI, PI32, c_long, PL, PI, PI]),
}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            path = _build.host_library_path() or _build.build_host(verbose=True)
            lib = ctypes.CDLL(path)
            lib.leone_host_last_error.restype = c_char_p
            lib.leone_host_last_error.argtypes = []
            for name, (restype, argtypes) in _PROTOTYPES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def last_error() -> str:
    return library().leone_host_last_error().decode("utf-8", "replace")
