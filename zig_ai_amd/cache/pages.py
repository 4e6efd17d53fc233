"""Pools of fixed-size things handed out and taken back: cache pages and state
slots.  Pure bookkeeping, no device memory.

The reference's allocator is a LIFO free list with reference counts, copy on
write and a CPU swap (/root/reference/src/paged_attention/allocator.zig:19-118);
this pool keeps the free list and replaces the reference count by a single
owner per page, which is all that requests that never share pages need, and
which makes "held twice" and "freed twice" detectable.
"""

from __future__ import annotations

from typing import Hashable, List, Optional


class OutOfPages(RuntimeError):
    """The pool cannot supply the pages asked for; nothing was taken."""


class OutOfSlots(RuntimeError):
    """Every state slot is in use."""


class PoolError(RuntimeError):
    """A bookkeeping invariant was violated (double free, foreign page, ...)."""


class Pool:
    """``size`` numbered items; ``take(owner)`` pops the most recently returned
    one, ``give(item, owner)`` returns it."""

    def __init__(self, size: int, what: str = "page"):
        if size < 0:
            raise ValueError(f"a pool cannot have {size} {what}s")
        self.size = size
        self.what = what
        self._free: List[int] = list(range(size - 1, -1, -1))   # pop() yields 0 first
        self._owner: List[Optional[Hashable]] = [None] * size
        self.high_water = 0
        self.total_taken = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return self.size - len(self._free)

    def take(self, owner: Hashable) -> int:
        if owner is None:
            raise PoolError("an owner is needed")
        if not self._free:
            raise (OutOfPages if self.what == "page" else OutOfSlots)(
                f"no free {self.what} (all {self.size} in use)")
        item = self._free.pop()
        if self._owner[item] is not None:
            raise PoolError(f"{self.what} {item} was on the free list while owned by "
                            f"{self._owner[item]!r}")
        self._owner[item] = owner
        self.total_taken += 1
        self.high_water = max(self.high_water, self.used_count)
        return item

    def take_many(self, owner: Hashable, n: int) -> List[int]:
        """All ``n`` or none."""
        if n > len(self._free):
            raise (OutOfPages if self.what == "page" else OutOfSlots)(
                f"{n} {self.what}s wanted, {len(self._free)} of {self.size} free")
        return [self.take(owner) for _ in range(n)]

    def give(self, item: int, owner: Hashable) -> None:
        if not 0 <= item < self.size:
            raise PoolError(f"{self.what} {item} does not exist")
        if self._owner[item] is None:
            raise PoolError(f"{self.what} {item} freed twice")
        if self._owner[item] != owner:
            raise PoolError(f"{self.what} {item} belongs to {self._owner[item]!r}, not {owner!r}")
        self._owner[item] = None
        self._free.append(item)

    def owner_of(self, item: int) -> Optional[Hashable]:
        return self._owner[item]

    def check(self) -> None:
        """Every item is either free exactly once or owned, never both."""
        seen = set()
        for item in self._free:
            if item in seen:
                raise PoolError(f"{self.what} {item} is on the free list twice")
            seen.add(item)
            if self._owner[item] is not None:
                raise PoolError(f"{self.what} {item} is free and owned")
        owned = sum(1 for o in self._owner if o is not None)
        if owned + len(self._free) != self.size:
            raise PoolError(f"{owned} owned + {len(self._free)} free != {self.size} {self.what}s")
