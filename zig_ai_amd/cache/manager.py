"""The cache manager: pages of keys and values for the mixers that need them,
with one block table per request and group, and one slot of fixed-size state
per request for the mixers that carry state.

Groups.  Mixers declare what they need (``PagedNeed`` or ``StateNeed``).  Paged
needs that are equal (the same planes per token, window and storage type) form a
*group*: its layers
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

Device memory: per group one tensor ``[layer, page, elements of a page]``; a page
holds the group's planes one after the other, plane ``p`` as ``[heads_p, page_size,
width_p]``, and every layer sees it as one view per plane.  For keys and values (two
planes of one size) that is the tensor ``kv[page, 2, kv_head, page_size, head_dim]``
the attention kernels take, where a page's keys lie as ``[offset][head_dim]`` and
the kernels store its values turned round as ``[head_dim][offset]`` (the order
their second product reads).  State: ``slots[slot, bytes]`` with one typed view per
state entry (32-bit floats unless the need says otherwise).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Mapping, Optional, Sequence, Tuple

import ctypes

import numpy as np
import torch

from ..kernels import host
from ..parts.base import PagedNeed, StateNeed
from .pages import Pool, raise_for

FREED = -1   # block-table entry of a page that was given back (behind the window)


@dataclass
class PagedGroup:
    index: int
    need: PagedNeed
    cache_ids: List[Hashable]
    pool: Pool
    page_size: int
    dtype: torch.dtype = torch.bfloat16
    memory: Optional[torch.Tensor] = None      # [layers, pages, elements of a page]

    def layer_of(self, cache_id) -> int:
        return self.cache_ids.index(cache_id)

    def elements_per_page(self) -> int:
        return self.need.elements_per_token() * self.page_size

    def bytes_per_page(self, element_size: Optional[int] = None) -> int:
        size = torch.empty((), dtype=self.dtype).element_size() if element_size is None else element_size
        return len(self.cache_ids) * self.elements_per_page() * size

    @property
    def kv(self) -> Optional[torch.Tensor]:
        """Keys and values of every layer, ``[layers, pages, 2, kv_heads, page_size,
        head_dim]``; only for a group of two equal planes."""
        if self.memory is None or not self.need.is_kv:
            return None
        heads, width = self.need.planes[0]
        return self.memory.view(len(self.cache_ids), self.pool.size, 2, heads, self.page_size, width)

    def plane_views(self, layer: int) -> List[torch.Tensor]:
        """One view ``[pages, heads, page_size, width]`` per plane of ``layer``."""
        if self.memory is None:
            return []
        mem = self.memory[layer]
        per_page = self.elements_per_page()
        out, offset = [], 0
        for heads, width in self.need.planes:
            n = heads * self.page_size * width
            out.append(mem[:, offset:offset + n].unflatten(1, (heads, self.page_size, width)))
            offset += n
        return out


@dataclass
class CacheView:
    """What a mixer sees of the cache for one entry of the run order."""
    kind: str                      # "paged" | "state" | "none"
    group: int = -1                # paged: index of the group (selects table and slots)
    kv: Optional[torch.Tensor] = None        # paged, keys and values: [pages, 2, kv_heads, page_size, head_dim]
    planes: Optional[List[torch.Tensor]] = None   # paged: per plane [pages, heads, page_size, width]
    state: Optional[torch.Tensor] = None     # state: [slots, *shape]
    writes: bool = True


class CacheManager:
    """Groups, tables and slots are kept by the host library; this class owns the
    device memory, names the requests and translates failures into exceptions."""

    def __init__(self, needs: Mapping[Hashable, object], page_size: int, num_pages, num_slots: int,
                 device: Optional[torch.device] = None, dtype: torch.dtype = torch.bfloat16,
                 allocate: bool = True, scatter_pages: bool = False):
        """``needs``: cache id -> PagedNeed | StateNeed | None.  ``num_pages``: an int
        (every group gets that many) or a mapping from the group's ``PagedNeed`` to a
        count.  ``scatter_pages``: fresh pools hand
        their pages out in a fixed pseudo-random order rather than 0, 1, 2 ..., so that
        requests filled one after the other do not lie a constant distance apart."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.device = device
        self.dtype = dtype
        self._lib = host.lib()
        self.handles = host.Handles()
        self._pinned: set = set()      # names a scheduler still knows: their handles are kept
        self._group_of: Dict[Hashable, int] = {}
        by_key: Dict[PagedNeed, int] = {}
        group_needs: List[PagedNeed] = []
        group_ids: List[List[Hashable]] = []
        group_pages: List[int] = []
        state_entries: List[Tuple[Hashable, StateNeed]] = []
        for cid, need in needs.items():
            if need is None:
                continue
            if isinstance(need, PagedNeed):
                if not need.planes or any(h <= 0 or w <= 0 for h, w in need.planes):
                    raise ValueError(f"cache entry {cid!r}: a paged need has planes of positive "
                                     f"sizes, got {need.planes!r}")
                if need not in by_key:
                    count = num_pages[need] if isinstance(num_pages, Mapping) else int(num_pages)
                    if count < 0:
                        raise ValueError(f"a pool cannot have {count} pages")
                    by_key[need] = len(group_needs)
                    group_needs.append(need)
                    group_ids.append([])
                    group_pages.append(count)
                group_ids[by_key[need]].append(cid)
                self._group_of[cid] = by_key[need]
            elif isinstance(need, StateNeed):
                state_entries.append((cid, need))
            else:
                raise TypeError(f"cache need of entry {cid!r} is {need!r}")
        if num_slots < 0:
            raise ValueError(f"a pool cannot have {num_slots} slots")
        G = len(group_needs)
        windows = (ctypes.c_int * max(G, 1))(*[n.window for n in group_needs])
        pages = (ctypes.c_int * max(G, 1))(*group_pages)
        self._ptr = self._lib.za_cache_new(G, windows, pages, int(page_size), int(num_slots),
                                           1 if scatter_pages else 0)
        if not self._ptr:
            raise ValueError("the host library refused the cache's sizes")
        self.groups: List[PagedGroup] = [
            PagedGroup(g, group_needs[g], group_ids[g],
                       Pool(0, "page", _attach=(self._lib.za_cache_pool(self._ptr, g), self.handles)),
                       page_size, group_needs[g].dtype or dtype)
            for g in range(G)]
        self.slots = Pool(0, "slot", _attach=(self._lib.za_cache_pool(self._ptr, -1), self.handles))
        # a slot is a row of bytes; every state entry has its own 16-byte aligned window of it
        self._state_layout: Dict[Hashable, Tuple[int, int, Tuple[int, ...], torch.dtype]] = {}
        offset = 0
        for cid, need in state_entries:
            n = 1
            for s in need.shape:
                n *= int(s)
            nbytes = n * torch.empty((), dtype=need.dtype).element_size()
            self._state_layout[cid] = (offset, nbytes, tuple(int(s) for s in need.shape), need.dtype)
            offset += (nbytes + 15) // 16 * 16
        self.bytes_per_slot = offset
        self.slot_memory: Optional[torch.Tensor] = None
        # what a new request's slot holds: zero bytes, or a row with every state entry's own
        # starting value (``StateNeed.init``)
        self._slot_start: Optional[torch.Tensor] = None
        if allocate:
            if device is None:
                raise ValueError("a device is needed to allocate the cache")
            for grp in self.groups:
                grp.memory = torch.zeros((len(grp.cache_ids), grp.pool.size, grp.elements_per_page()),
                                         dtype=grp.dtype, device=device)
            if self.bytes_per_slot:
                self.slot_memory = torch.zeros((num_slots, self.bytes_per_slot),
                                               dtype=torch.uint8, device=device)
                if any(need.init != 0 for _, need in state_entries):
                    start = torch.zeros((self.bytes_per_slot,), dtype=torch.uint8, device=device)
                    for cid, need in state_entries:
                        if need.init != 0:
                            off, nbytes, _, dt = self._state_layout[cid]
                            start[off:off + nbytes].view(dt).fill_(need.init)
                    self._slot_start = start
        self._n_groups = G
        self._scratch = (ctypes.c_int * max(G, 1))()

    def __del__(self):
        ptr, self._ptr = getattr(self, "_ptr", None), None
        if ptr:
            self._lib.za_cache_free(ptr)

    @property
    def native(self) -> int:
        """The host library's object, for the scheduler and the step builder."""
        return self._ptr

    @staticmethod
    def bytes_per_page_index(needs: Mapping[Hashable, object], page_size: int,
                             run_dtype: torch.dtype) -> int:
        """Device bytes that ONE more page in every group costs (all groups are given
        the same number of pages when ``num_pages`` is a single number)."""
        total = 0
        for need in needs.values():
            if isinstance(need, PagedNeed):
                size = torch.empty((), dtype=need.dtype or run_dtype).element_size()
                total += need.elements_per_token() * page_size * size
        return total

    # ------------------------------------------------------------------ views
    def view(self, cache_id, writes: bool = True) -> CacheView:
        if cache_id in self._group_of:
            grp = self.groups[self._group_of[cache_id]]
            layer = grp.layer_of(cache_id)
            kv = grp.kv[layer] if grp.kv is not None else None
            return CacheView("paged", group=grp.index, kv=kv, planes=grp.plane_views(layer),
                             writes=writes)
        if cache_id in self._state_layout:
            off, nbytes, shape, dtype = self._state_layout[cache_id]
            st = None
            if self.slot_memory is not None:
                # A window of every slot's row: contiguous within a slot, slots spaced by
                # the whole row.
                st = self.slot_memory[:, off:off + nbytes].view(dtype).unflatten(1, shape)
            return CacheView("state", state=st, writes=writes)
        return CacheView("none", writes=writes)

    # --------------------------------------------------------------- requests
    def _info(self, req: Hashable):
        h = self.handles.known(req)
        out = (ctypes.c_longlong * 4)()
        if h is None or not self._lib.za_cache_request(self._ptr, h, out):
            raise KeyError(req)
        return out

    def __contains__(self, req: Hashable) -> bool:
        h = self.handles.known(req)
        out = (ctypes.c_longlong * 4)()
        return h is not None and bool(self._lib.za_cache_request(self._ptr, h, out))

    @property
    def requests(self):
        """The admitted requests' names (a container: ``in``, ``len``)."""
        return _Admitted(self)

    def pin(self, req: Hashable) -> int:
        """Keep the request's handle until ``unpin`` (for a scheduler that knows the
        request also while it is not admitted)."""
        self._pinned.add(req)
        return self.handles.of(req)

    def unpin(self, req: Hashable) -> None:
        self._pinned.discard(req)
        if req not in self:
            self.handles.drop(req)

    def admit(self, req: Hashable) -> int:
        slot = ctypes.c_int()
        raise_for(self._lib.za_cache_admit(self._ptr, self.handles.of(req), ctypes.byref(slot)))
        self._start_slot(slot.value)
        return slot.value

    def _start_slot(self, slot: int) -> None:
        """A new request's state: every entry at its starting value."""
        if self.slot_memory is None:
            return
        if self._slot_start is None:
            self.slot_memory[slot].zero_()
        else:
            self.slot_memory[slot].copy_(self._slot_start)

    def admitted_by_scheduler(self, req: Hashable) -> None:
        """The host library's scheduler admitted ``req`` itself: start its state."""
        self._start_slot(self.slot_of(req))

    def pages_needed(self, req: Hashable, n_new: int) -> Dict[int, int]:
        if req not in self:
            raise KeyError(req)
        raise_for(self._lib.za_cache_pages_needed(self._ptr, self.handles.of(req), int(n_new),
                                                  self._scratch))
        return {g: self._scratch[g] for g in range(self._n_groups)}

    def can_reserve(self, req: Hashable, n_new: int, spare: Optional[Dict[int, int]] = None) -> bool:
        """Whether ``reserve`` would succeed; ``spare`` (group -> pages) is
        subtracted from the free counts first (pages promised to others)."""
        if req not in self:
            raise KeyError(req)
        sp = None
        if spare:
            sp = (ctypes.c_int * max(self._n_groups, 1))(
                *[int(spare.get(g, 0)) for g in range(self._n_groups)])
        ok = ctypes.c_int()
        raise_for(self._lib.za_cache_can_reserve(self._ptr, self.handles.of(req), int(n_new), sp,
                                                 ctypes.byref(ok)))
        return bool(ok.value)

    def reserve(self, req: Hashable, n_new: int) -> None:
        """Make the request's tables cover ``n_new`` more tokens; all groups or none."""
        if req not in self:
            raise KeyError(req)
        raise_for(self._lib.za_cache_reserve(self._ptr, self.handles.of(req), int(n_new)))

    def commit(self, req: Hashable, n_new: int) -> None:
        """``n_new`` tokens were written; give back pages no later query can read."""
        if req not in self:
            raise KeyError(req)
        raise_for(self._lib.za_cache_commit(self._ptr, self.handles.of(req), int(n_new)))

    def reserve_many(self, reqs: Sequence[Hashable], counts: Sequence[int]) -> None:
        """Pages for every entry of a step, all of them or none.  Raises ``KeyError``
        for a request that is not admitted."""
        h = np.empty((len(reqs),), dtype=np.int64)
        for i, r in enumerate(reqs):
            known = self.handles.known(r)
            if known is None:
                raise KeyError(r)
            h[i] = known
        c = np.asarray(counts, dtype=np.int32)
        rc = self._lib.za_cache_reserve_many(self._ptr, len(reqs), h.ctypes.data, c.ctypes.data)
        if rc == host.STEP:
            raise KeyError(reqs[int(host.last_error().split()[1].rstrip(":"))])
        raise_for(rc)

    def commit_many(self, reqs: Sequence[Hashable], counts: Sequence[int]) -> None:
        h = np.fromiter((self.handles.of(r) for r in reqs), dtype=np.int64, count=len(reqs))
        c = np.asarray(counts, dtype=np.int32)
        raise_for(self._lib.za_cache_commit_many(self._ptr, len(reqs), h.ctypes.data, c.ctypes.data))

    def release(self, req: Hashable) -> None:
        if req not in self:
            raise KeyError(req)
        raise_for(self._lib.za_cache_release(self._ptr, self.handles.of(req)))
        if req not in self._pinned:
            self.handles.drop(req)

    # ------------------------------------------------------------- step inputs
    def slot_of(self, req: Hashable) -> int:
        return int(self._info(req)[0])

    def num_tokens(self, req: Hashable) -> int:
        return int(self._info(req)[1])

    def serial_of(self, req: Hashable) -> int:
        """A number that differs between two admissions, also of the same id."""
        return int(self._info(req)[3])

    def table(self, req: Hashable, group: int) -> List[int]:
        if req not in self:
            raise KeyError(req)
        h = self.handles.of(req)
        n = self._lib.za_cache_table(self._ptr, h, int(group), None, 0)
        if n < 0:
            raise KeyError((req, group))
        out = np.empty((max(n, 1),), dtype=np.int32)
        self._lib.za_cache_table(self._ptr, h, int(group), out.ctypes.data, n)
        return out[:n].tolist()

    def token_slots(self, req: Hashable, group: int, start: int, n: int) -> List[int]:
        """Physical places ``page * page_size + offset`` of positions start..start+n-1."""
        if req not in self:
            raise KeyError(req)
        out = np.empty((max(n, 1),), dtype=np.int32)
        raise_for(self._lib.za_cache_token_slots(self._ptr, self.handles.of(req), int(group),
                                                 int(start), int(n), out.ctypes.data))
        return out[:n].tolist()

    # ------------------------------------------------------------------ checks
    def check(self) -> None:
        """No page lost, held twice or freed twice; tables agree with the pools."""
        raise_for(self._lib.za_cache_check(self._ptr))

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

    @property
    def pages_reused(self) -> int:
        return int(self._lib.za_cache_pages_reused(self._ptr))


class _Admitted:
    """``cache.requests``: which names are admitted."""

    def __init__(self, cache: "CacheManager"):
        self._cache = cache

    def __contains__(self, req: Hashable) -> bool:
        return req in self._cache

    def __len__(self) -> int:
        return int(self._cache._lib.za_cache_num_requests(self._cache._ptr))
