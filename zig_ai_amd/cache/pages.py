"""Pools of fixed-size things handed out and taken back: cache pages and state
slots.  Pure bookkeeping, no device memory; the free list and the owners live in
the host library (``csrc/host.cpp``), this class is its Python face.

The reference's allocator is a LIFO free list with reference counts, copy on
write and a CPU swap (/root/reference/src/paged_attention/allocator.zig:19-118);
this pool keeps the free list and replaces the reference count by a single
owner per page, which is all that requests that never share pages need, and
which makes "held twice" and "freed twice" detectable.
"""

from __future__ import annotations

import ctypes
from typing import Hashable, List, Optional

from ..kernels import host


class OutOfPages(RuntimeError):
    """The pool cannot supply the pages asked for; nothing was taken."""


class OutOfSlots(RuntimeError):
    """Every state slot is in use."""


class PoolError(RuntimeError):
    """A bookkeeping invariant was violated (double free, foreign page, ...)."""


def raise_for(code: int) -> None:
    """Turn a failure code of the host library into this package's exception."""
    if code == host.OK:
        return
    msg = host.last_error()
    if code == host.OUT_OF_PAGES:
        raise OutOfPages(msg)
    if code == host.OUT_OF_SLOTS:
        raise OutOfSlots(msg)
    if code == host.POOL:
        raise PoolError(msg)
    if code == host.ARG:
        raise ValueError(msg)
    raise RuntimeError(f"host library error {code}: {msg}")


class Pool:
    """``size`` numbered items; ``take(owner)`` pops the most recently returned
    one, ``give(item, owner)`` returns it."""

    def __init__(self, size: int, what: str = "page", _attach=None):
        """``_attach``: ``(pointer, handles)`` of a pool that a cache owns."""
        self.what = what
        self._lib = host.lib()
        if _attach is not None:
            self._ptr, self._handles = _attach
            self._own = False
        else:
            if size < 0:
                raise ValueError(f"a pool cannot have {size} {what}s")
            self._ptr = self._lib.za_pool_new(int(size), 1 if what == "page" else 0)
            self._handles = host.Handles()
            self._own = True
        self.size = self._stats()[0]

    def __del__(self):
        if getattr(self, "_own", False) and self._ptr:
            self._lib.za_pool_free(self._ptr)
            self._ptr = None

    def _stats(self):
        out = (ctypes.c_longlong * 4)()
        self._lib.za_pool_stats(self._ptr, out)
        return list(out)

    @property
    def free_count(self) -> int:
        return self._stats()[1]

    @property
    def used_count(self) -> int:
        s = self._stats()
        return s[0] - s[1]

    @property
    def high_water(self) -> int:
        return self._stats()[2]

    @property
    def total_taken(self) -> int:
        return self._stats()[3]

    def take(self, owner: Hashable) -> int:
        if owner is None:
            raise PoolError("an owner is needed")
        item = ctypes.c_int()
        raise_for(self._lib.za_pool_take(self._ptr, self._handles.of(owner), ctypes.byref(item)))
        return item.value

    def take_many(self, owner: Hashable, n: int) -> List[int]:
        """All ``n`` or none."""
        if owner is None:
            raise PoolError("an owner is needed")
        items = (ctypes.c_int * max(n, 1))()
        raise_for(self._lib.za_pool_take_many(self._ptr, self._handles.of(owner), int(n), items))
        return list(items[:n])

    def give(self, item: int, owner: Hashable) -> None:
        known = self._handles.known(owner)
        raise_for(self._lib.za_pool_give(self._ptr, int(item), known if known is not None else 0))

    def owner_of(self, item: int) -> Optional[Hashable]:
        owner = ctypes.c_int64()
        if self._lib.za_pool_owner(self._ptr, int(item), ctypes.byref(owner)) == 1:
            return self._handles.name(owner.value)
        return None

    def check(self) -> None:
        """Every item is either free exactly once or owned, never both."""
        raise_for(self._lib.za_pool_check(self._ptr))
