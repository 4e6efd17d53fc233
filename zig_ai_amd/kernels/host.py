"""ctypes declarations of the host-side library (``csrc/host.cpp``): pools, block
tables, the scheduler's decisions, the step's integer buffer, uniform streams.

The classes that the rest of the package uses (``cache.Pool``, ``cache.CacheManager``,
``engine.Scheduler``, ``engine.build_step``, ``sampling.UniformStream``) keep their
requests' names (any hashable) on the Python side and hand the library 64-bit
handles; ``Handles`` is that table.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int64, c_longlong, c_void_p
from typing import Dict, Hashable, Optional

from . import build

OK, OUT_OF_PAGES, OUT_OF_SLOTS, POOL, ARG, STEP = 0, 1, 2, 3, 4, 5

_P = POINTER
_SIGNATURES = {
    "za_host_last_error": (c_char_p, []),
    "za_pool_new": (c_void_p, [c_int, c_int]),
    "za_pool_free": (None, [c_void_p]),
    "za_pool_take": (c_int, [c_void_p, c_int64, _P(c_int)]),
    "za_pool_take_many": (c_int, [c_void_p, c_int64, c_int, _P(c_int)]),
    "za_pool_give": (c_int, [c_void_p, c_int, c_int64]),
    "za_pool_check": (c_int, [c_void_p]),
    "za_pool_stats": (None, [c_void_p, _P(c_longlong)]),
    "za_pool_owner": (c_int, [c_void_p, c_int, _P(c_int64)]),
    "za_cache_new": (c_void_p, [c_int, _P(c_int), _P(c_int), c_int, c_int, c_int]),
    "za_cache_free": (None, [c_void_p]),
    "za_cache_pool": (c_void_p, [c_void_p, c_int]),
    "za_cache_admit": (c_int, [c_void_p, c_int64, _P(c_int)]),
    "za_cache_pages_needed": (c_int, [c_void_p, c_int64, c_int, _P(c_int)]),
    "za_cache_can_reserve": (c_int, [c_void_p, c_int64, c_int, _P(c_int), _P(c_int)]),
    "za_cache_reserve": (c_int, [c_void_p, c_int64, c_int]),
    "za_cache_commit": (c_int, [c_void_p, c_int64, c_int]),
    "za_cache_release": (c_int, [c_void_p, c_int64]),
    "za_cache_reserve_many": (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    "za_cache_commit_many": (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    "za_cache_request": (c_int, [c_void_p, c_int64, _P(c_longlong)]),
    "za_cache_num_requests": (c_int, [c_void_p]),
    "za_cache_pages_reused": (c_longlong, [c_void_p]),
    "za_cache_table": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_int]),
    "za_cache_token_slots": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "za_cache_check": (c_int, [c_void_p]),
    "za_step_build": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_longlong,
                              c_void_p, c_void_p, c_void_p, c_void_p]),
    "za_decode_prepare": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "za_sched_new": (c_void_p, [c_void_p, c_int, c_int, c_int, c_int]),
    "za_sched_free": (None, [c_void_p]),
    "za_sched_add": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, c_int, _P(c_longlong)]),
    "za_sched_forget": (c_int, [c_void_p, c_int64]),
    "za_sched_abort": (c_int, [c_void_p, c_int64]),
    "za_sched_has_work": (c_int, [c_void_p]),
    "za_sched_schedule": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  _P(c_int), c_void_p, _P(c_int)]),
    "za_sched_update": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_void_p, _P(c_int)]),
    "za_sched_request": (c_int, [c_void_p, c_int64, _P(c_longlong)]),
    "za_sched_queue": (c_int, [c_void_p, c_int, c_void_p, c_int]),
    "za_sched_preemptions": (c_longlong, [c_void_p]),
    "za_uniforms": (None, [c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
}

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The host library with its functions declared (compiled at first use)."""
    global _lib
    if _lib is None:
        loaded = build.load("host")
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(loaded, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = loaded
    return _lib


def last_error() -> str:
    return lib().za_host_last_error().decode("utf-8", "replace")


class Handles:
    """Names of requests (any hashable) <-> the 64-bit numbers the library knows
    them by.  A name keeps its number until it is dropped."""

    def __init__(self) -> None:
        self._of: Dict[Hashable, int] = {}
        self._name: Dict[int, Hashable] = {}
        self._next = 1

    def of(self, name: Hashable) -> int:
        h = self._of.get(name)
        if h is None:
            h = self._next
            self._next += 1
            self._of[name] = h
            self._name[h] = name
        return h

    def known(self, name: Hashable) -> Optional[int]:
        return self._of.get(name)

    def name(self, handle: int) -> Hashable:
        return self._name[handle]

    def drop(self, name: Hashable) -> None:
        h = self._of.pop(name, None)
        if h is not None:
            del self._name[h]

    def __len__(self) -> int:
        return len(self._of)
