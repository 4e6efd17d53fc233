"""The cache manager: pages of keys and values for the mixers that need them,
with one block table per request and group, and one slot of fixed-size state
per request for the mixers that carry state.

Groups.  Mixers declare what they need (``PagedNeed`` or ``StateNeed``).  Paged
needs with the same (kv heads, head size, window) form a *group*: its layers
share one block table per request (page ``p`` names the same place in every
layer's plane of the group's tensor) and the group has a pool of pages of its
own, because a group that keeps every key and a group that keeps a window of
keys fill and empty at different rates.  The reference instead gives each
attention layer its own table over one shared pool and keeps recurrent state
inside the layer object, which limits it to one live request
(/root/reference/src/main.zig:687-696, /root/reference/src/transformer/short_conv.zig:63-64).

Life of a request: ``admit`` (takes a slot, zeroes its state), then per step
``reserve`` (pages for the step's tokens; all or nothing) and ``commit`` (the
tokens are in the cache; pages wholly behind a group's window go back to the
pool), finally ``release`` (every page and the slot go back).

Device memory: per group ``kv[layer, page, 2, kv_head, page_size * head_dim]``,
where a page's keys lie as ``[offset][head_dim]`` and its values turned round as
``[head_dim][offset]`` (the order the attention kernels' second product reads);
state ``slots[slot, floats]`` in 32-bit with one view per state entry.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Mapping, Optional, Tuple

import torch

from ..parts.base import PagedNeed, StateNeed
from .pages import OutOfPages, OutOfSlots, Pool, PoolError

FREED = -1   # block-table entry of a page that was given back (behind the window)


@dataclass
class PagedGroup:
    index: int
    need: PagedNeed
    cache_ids: List[int]
    pool: Pool
    page_size: int
    kv: Optional[torch.Tensor] = None      # [layers, pages, 2, kv_heads, page_size, head_dim]

    def layer_of(self, cache_id: int) -> int:
        return self.cache_ids.index(cache_id)

    def bytes_per_page(self, element_size: int) -> int:
        n = self.need
        return len(self.cache_ids) * 2 * n.num_kv_heads * self.page_size * n.head_dim * element_size


@dataclass
class RequestCache:
    slot: int
    num_tokens: int = 0
    tables: Dict[int, List[int]] = field(default_factory=dict)   # group index -> page ids
    reserved: int = 0                                            # tokens the tables cover
    serial: int = 0                                              # number of this admission


@dataclass
class CacheView:
    """What a mixer sees of the cache for one entry of the run order."""
    kind: str                      # "paged" | "state" | "none"
    group: int = -1                # paged: index of the group (selects table and slots)
    kv: Optional[torch.Tensor] = None        # paged: [pages, 2, kv_heads, page_size, head_dim]
    state: Optional[torch.Tensor] = None     # state: [slots, *shape]
    writes: bool = True


class CacheManager:
    def __init__(self, needs: Mapping[int, object], page_size: int, num_pages, num_slots: int,
                 device: Optional[torch.device] = None, dtype: torch.dtype = torch.bfloat16,
                 allocate: bool = True):
        """``needs``: cache id -> PagedNeed | StateNeed | None.  ``num_pages``: an int
        (every group gets that many) or a mapping from group key
        ``(kv_heads, head_dim, window)`` to a count."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.device = device
        self.dtype = dtype
        self.groups: List[PagedGroup] = []
        self._group_of: Dict[int, int] = {}
        by_key: Dict[Tuple[int, int, int], PagedGroup] = {}
        state_entries: List[Tuple[int, StateNeed]] = []
        for cid in sorted(needs):
            need = needs[cid]
            if need is None:
                continue
            if isinstance(need, PagedNeed):
                key = (need.num_kv_heads, need.head_dim, need.window)
                if key not in by_key:
                    count = num_pages[key] if isinstance(num_pages, Mapping) else int(num_pages)
                    grp = PagedGroup(len(self.groups), need, [], Pool(count, "page"), page_size)
                    by_key[key] = grp
                    self.groups.append(grp)
                by_key[key].cache_ids.append(cid)
                self._group_of[cid] = by_key[key].index
            elif isinstance(need, StateNeed):
                state_entries.append((cid, need))
            else:
                raise TypeError(f"cache need of entry {cid} is {need!r}")
        self.slots = Pool(num_slots, "slot")
        self._state_layout: Dict[int, Tuple[int, Tuple[int, ...]]] = {}
        offset = 0
        for cid, need in state_entries:
            n = 1
            for s in need.shape:
                n *= int(s)
            self._state_layout[cid] = (offset, tuple(int(s) for s in need.shape))
            offset += n
        self.floats_per_slot = offset
        self.slot_memory: Optional[torch.Tensor] = None
        if allocate:
            if device is None:
                raise ValueError("a device is needed to allocate the cache")
            for grp in self.groups:
                n = grp.need
                grp.kv = torch.zeros((len(grp.cache_ids), grp.pool.size, 2, n.num_kv_heads,
                                      page_size, n.head_dim), dtype=dtype, device=device)
            if self.floats_per_slot:
                self.slot_memory = torch.zeros((num_slots, self.floats_per_slot),
                                               dtype=torch.float32, device=device)
        self.requests: Dict[Hashable, RequestCache] = {}
        self.pages_reused = 0
        self._admissions = 0
        self._ever_used: List[set] = [set() for _ in self.groups]

    # ------------------------------------------------------------------ views
    def view(self, cache_id: int, writes: bool = True) -> CacheView:
        if cache_id in self._group_of:
            grp = self.groups[self._group_of[cache_id]]
            kv = grp.kv[grp.layer_of(cache_id)] if grp.kv is not None else None
            return CacheView("paged", group=grp.index, kv=kv, writes=writes)
        if cache_id in self._state_layout:
            off, shape = self._state_layout[cache_id]
            st = None
            if self.slot_memory is not None:
                n = 1
                for s in shape:
                    n *= s
                # A window of every slot's row: contiguous within a slot, slots spaced by
                # the whole row.
                st = self.slot_memory[:, off:off + n].unflatten(1, shape)
            return CacheView("state", state=st, writes=writes)
        return CacheView("none", writes=writes)

    # --------------------------------------------------------------- requests
    def admit(self, req: Hashable) -> int:
        if req in self.requests:
            raise PoolError(f"request {req!r} is already admitted")
        slot = self.slots.take(req)
        self._admissions += 1
        self.requests[req] = RequestCache(slot, 0, {g.index: [] for g in self.groups}, 0,
                                          self._admissions)
        if self.slot_memory is not None:
            self.slot_memory[slot].zero_()
        return slot

    def pages_needed(self, req: Hashable, n_new: int) -> Dict[int, int]:
        rc = self.requests[req]
        total = rc.num_tokens + n_new
        want = (total + self.page_size - 1) // self.page_size
        return {g.index: max(0, want - len(rc.tables[g.index])) for g in self.groups}

    def can_reserve(self, req: Hashable, n_new: int, spare: Optional[Dict[int, int]] = None) -> bool:
        """Whether ``reserve`` would succeed; ``spare`` (group -> pages) is
        subtracted from the free counts first (pages promised to others)."""
        for gi, n in self.pages_needed(req, n_new).items():
            free = self.groups[gi].pool.free_count - (spare or {}).get(gi, 0)
            if n > free:
                return False
        return True

    def reserve(self, req: Hashable, n_new: int) -> None:
        """Make the request's tables cover ``n_new`` more tokens; all groups or none."""
        rc = self.requests[req]
        needed = self.pages_needed(req, n_new)
        for gi, n in needed.items():
            if n > self.groups[gi].pool.free_count:
                raise OutOfPages(
                    f"request {req!r} needs {n} pages of group {gi}, "
                    f"{self.groups[gi].pool.free_count} of {self.groups[gi].pool.size} free")
        for gi, n in needed.items():
            pool = self.groups[gi].pool
            for _ in range(n):
                page = pool.take(req)
                if page in self._ever_used[gi]:
                    self.pages_reused += 1
                self._ever_used[gi].add(page)
                rc.tables[gi].append(page)
        rc.reserved = max(rc.reserved, rc.num_tokens + n_new)

    def commit(self, req: Hashable, n_new: int) -> None:
        """``n_new`` tokens were written; give back pages no later query can read."""
        rc = self.requests[req]
        if rc.num_tokens + n_new > rc.reserved:
            raise PoolError(f"request {req!r} commits {n_new} tokens beyond its reservation")
        rc.num_tokens += n_new
        for grp in self.groups:
            w = grp.need.window
            if w <= 0:
                continue
            # The next query sits at position >= num_tokens and reads keys > position - w.
            first_needed = rc.num_tokens - w + 1
            if first_needed <= 0:
                continue
            table = rc.tables[grp.index]
            for p in range(min(first_needed // self.page_size, len(table))):
                if table[p] != FREED:
                    grp.pool.give(table[p], req)
                    table[p] = FREED

    def release(self, req: Hashable) -> None:
        rc = self.requests.pop(req)
        for grp in self.groups:
            for page in rc.tables[grp.index]:
                if page != FREED:
                    grp.pool.give(page, req)
        self.slots.give(rc.slot, req)

    # ------------------------------------------------------------- step inputs
    def slot_of(self, req: Hashable) -> int:
        return self.requests[req].slot

    def num_tokens(self, req: Hashable) -> int:
        return self.requests[req].num_tokens

    def serial_of(self, req: Hashable) -> int:
        """A number that differs between two admissions, also of the same id."""
        return self.requests[req].serial

    def table(self, req: Hashable, group: int) -> List[int]:
        return self.requests[req].tables[group]

    def token_slots(self, req: Hashable, group: int, start: int, n: int) -> List[int]:
        """Physical places ``page * page_size + offset`` of positions start..start+n-1."""
        table = self.requests[req].tables[group]
        ps = self.page_size
        out = []
        for pos in range(start, start + n):
            page = table[pos // ps]
            if page == FREED:
                raise PoolError(f"position {pos} of request {req!r} lies in a page given back")
            out.append(page * ps + pos % ps)
        return out

    # ------------------------------------------------------------------ checks
    def check(self) -> None:
        """No page lost, held twice or freed twice; tables agree with the pools."""
        self.slots.check()
        seen_slots = set()
        for req, rc in self.requests.items():
            if rc.slot in seen_slots:
                raise PoolError(f"slot {rc.slot} held twice")
            seen_slots.add(rc.slot)
            if self.slots.owner_of(rc.slot) != req:
                raise PoolError(f"slot {rc.slot} of {req!r} is owned by {self.slots.owner_of(rc.slot)!r}")
        if len(seen_slots) != self.slots.used_count:
            raise PoolError("slots in use do not match the admitted requests")
        for grp in self.groups:
            grp.pool.check()
            held = set()
            for req, rc in self.requests.items():
                for page in rc.tables[grp.index]:
                    if page == FREED:
                        continue
                    if page in held:
                        raise PoolError(f"page {page} of group {grp.index} held twice")
                    held.add(page)
                    if grp.pool.owner_of(page) != req:
                        raise PoolError(f"page {page} of {req!r} is owned by "
                                        f"{grp.pool.owner_of(page)!r}")
            if len(held) != grp.pool.used_count:
                raise PoolError(f"group {grp.index}: {grp.pool.used_count} pages in use but "
                                f"{len(held)} in tables (page lost)")

    def stats(self) -> dict:
        return {
            "groups": [{"window": g.need.window, "layers": len(g.cache_ids),
                        "pages": g.pool.size, "pages_free": g.pool.free_count,
                        "pages_high_water": g.pool.high_water,
                        "pages_taken": g.pool.total_taken} for g in self.groups],
            "slots": self.slots.size, "slots_free": self.slots.free_count,
            "slots_high_water": self.slots.high_water,
            "pages_reused": self.pages_reused, "requests": len(self.requests),
        }
