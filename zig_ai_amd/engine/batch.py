"""The description of one step that the model's parts read: which tokens, whose
they are, where they sit in their requests, and where their cache lives.

A step packs the new tokens of all its requests into one row sequence
``[T]``: request 0's tokens, then request 1's, and so on.  A request contributes
a portion of its prompt (one token or many) or one decoded token; the model does
not distinguish the two.  Every integer array the kernels need is laid out in
ONE host buffer (filled by the host library, ``csrc/host.cpp``) and copied to the
device in one transfer.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.pages import raise_for
from ..kernels import host as hostlib


class StepError(ValueError):
    """The entries of a step are malformed (empty, duplicated, out of range)."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()      # indices into ``tokens`` whose logits are returned


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    n_logit_rows: int
    max_keys: int                         # longest context (cached + new) in the step
    token_ids: torch.Tensor               # int32 [T]
    positions: torch.Tensor               # int32 [T]   position of each token in its request
    token_seq: torch.Tensor               # int32 [T]   index of the token's request in the step
    seq_start: torch.Tensor               # int32 [S+1] first row of each request, then T
    ctx_len: torch.Tensor                 # int32 [S]   tokens cached before this step
    slot_id: torch.Tensor                 # int32 [S]   state slot of each request
    logit_rows: torch.Tensor              # int32 [R]   rows whose logits are wanted
    block_tables: Dict[int, torch.Tensor] = field(default_factory=dict)   # group -> [S, max_pages]
    slot_mapping: Dict[int, torch.Tensor] = field(default_factory=dict)   # group -> [T]
    items: Dict[int, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]] = field(default_factory=dict)
    # host copies, for parts written in plain torch and for planning
    seq_lens_host: List[int] = field(default_factory=list)
    ctx_lens_host: List[int] = field(default_factory=list)
    slots_host: List[int] = field(default_factory=list)
    # the host image of the integer buffer and where each array sits in it
    host: Optional[np.ndarray] = None
    offsets: Dict[str, Tuple[int, int]] = field(default_factory=dict)
    table_width: int = 0
    # diagnostics: when a dict, the part that is running may leave copies of its
    # intermediate tensors in it by name (token rows first); see DecoderModel.forward
    taps: Optional[Dict[str, torch.Tensor]] = None

    def attention_items(self, rows_per_item: int):
        """Work items of at most ``rows_per_item`` consecutive query rows of one
        request: (request index, first row, row count) arrays and their number."""
        if rows_per_item not in self.items:
            seq, row0, cnt = _make_items(self.seq_lens_host, rows_per_item)
            dev = self.token_ids.device
            self.items[rows_per_item] = (
                torch.tensor(seq, dtype=torch.int32, device=dev),
                torch.tensor(row0, dtype=torch.int32, device=dev),
                torch.tensor(cnt, dtype=torch.int32, device=dev), len(seq))
        return self.items[rows_per_item]


def _make_items(seq_lens: Sequence[int], rows_per_item: int):
    seq, row0, cnt = [], [], []
    row = 0
    for s, n in enumerate(seq_lens):
        done = 0
        while done < n:
            c = min(rows_per_item, n - done)
            seq.append(s)
            row0.append(row + done)
            cnt.append(c)
            done += c
        row += n
    return seq, row0, cnt


class PreparedEntries:
    """The entries of a step as the arrays the host library reads."""

    def __init__(self, entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int):
        if not entries:
            raise StepError("a step needs at least one entry")
        S = len(entries)
        self.entries = entries
        self.reqs = np.empty((S,), dtype=np.int64)
        self.counts = np.empty((S,), dtype=np.int32)
        self.want_counts = np.empty((S,), dtype=np.int32)
        handles = cache.handles
        for s, e in enumerate(entries):
            h = handles.known(e.request)
            if h is None:
                raise StepError(f"request {e.request!r} is not admitted")
            self.reqs[s] = h
            self.counts[s] = len(e.tokens)
            self.want_counts[s] = len(e.want)
        try:
            # (a list of integers becomes an array at some 20 ns an element; a generator
            # over the tokens of a long portion costs five times that)
            tokens = self._integers([e.tokens for e in entries], int(self.counts.sum()))
            wants = self._integers([e.want for e in entries], int(self.want_counts.sum()))
        except (TypeError, ValueError, OverflowError) as err:
            raise StepError(f"token ids and wanted places must be integers: {err}") from err
        if tokens.size and (tokens.min() < 0 or tokens.max() >= vocab_size):
            where = int(np.flatnonzero((tokens < 0) | (tokens >= vocab_size))[0])
            owner = int(np.searchsorted(np.cumsum(self.counts), where, side="right"))
            raise StepError(f"request {entries[owner].request!r}: token id {int(tokens[where])} "
                            f"is outside the vocabulary of {vocab_size}")
        self.tokens = tokens.astype(np.int32)
        self.wants = np.clip(wants, -1, 2 ** 31 - 1).astype(np.int32)
        self.vocab_size = int(vocab_size)
        self.ctx = np.empty((S,), dtype=np.int32)
        self.slots = np.empty((S,), dtype=np.int32)
        self.meta = np.zeros((6,), dtype=np.int64)

    @staticmethod
    def _integers(parts: Sequence[Sequence[int]], total: int) -> np.ndarray:
        out = np.empty((total,), dtype=np.int64)
        at = 0
        for p in parts:
            n = len(p)
            if n:
                a = np.asarray(p)
                if a.dtype.kind not in "iu" or a.shape != (n,):
                    if a.dtype.kind == "b" or a.shape != (n,) or \
                            not all(isinstance(v, (int, np.integer)) and not isinstance(v, bool) for v in p):
                        raise TypeError(f"not integers: {p!r:.60}")
                    a = np.asarray([int(v) for v in p], dtype=np.int64)
                out[at:at + n] = a
                at += n
        return out

    def build(self, cache: CacheManager, grans: np.ndarray, max_position: int, min_pages: int,
              sections: np.ndarray, out_ptr, cap: int) -> None:
        """One call of the host library: with ``out_ptr`` None only the sizes."""
        rc = hostlib.lib().za_step_build(
            cache.native, len(self.entries), self.reqs.ctypes.data, self.counts.ctypes.data,
            self.tokens.ctypes.data, self.want_counts.ctypes.data, self.wants.ctypes.data,
            self.vocab_size, len(grans), grans.ctypes.data, int(max_position), int(min_pages),
            out_ptr, cap, sections.ctypes.data, self.meta.ctypes.data, self.ctx.ctypes.data,
            self.slots.ctypes.data)
        if rc == hostlib.STEP:
            msg = hostlib.last_error()
            if msg.startswith("entry "):        # name the request instead of its place
                place = int(msg.split()[1].rstrip(":"))
                msg = f"request {self.entries[place].request!r}: " + msg.split(" ", 2)[2]
            raise StepError(msg)
        raise_for(rc)


class StagingRing:
    """A few pinned host buffers that take turns: a step is laid out in one of them and
    goes to the device by a copy that does not block, so the host can lay out and issue the
    next step while this one still runs (a copy from ordinary memory makes the host wait
    for everything issued before it).  A buffer is used again only after its copy has
    finished (an event per buffer)."""

    def __init__(self, buffers: int = 4, words: int = 1 << 14):
        self._buffers: List[Optional[torch.Tensor]] = [None] * buffers
        self._events: List[Optional[torch.cuda.Event]] = [None] * buffers
        self._words = words
        self._at = -1

    def take(self, words: int) -> torch.Tensor:
        """A pinned int32 buffer of at least ``words`` entries, free to be written."""
        self._at = (self._at + 1) % len(self._buffers)
        ev = self._events[self._at]
        if ev is not None:
            ev.synchronize()
        buf = self._buffers[self._at]
        if buf is None or buf.numel() < words:
            buf = torch.empty((max(self._words, 2 * words),), dtype=torch.int32, pin_memory=True)
            self._buffers[self._at] = buf
        return buf

    def copied(self) -> None:
        """The copy out of the buffer taken last has been issued on the current stream."""
        if self._events[self._at] is None:
            self._events[self._at] = torch.cuda.Event()
        self._events[self._at].record()


def build_step(entries: Sequence[StepEntry], cache: CacheManager, device: torch.device,
               vocab_size: int, item_granularities: Sequence[int] = (),
               max_position: int = 0, min_pages: int = 0, max_keys: int = 0,
               into: Optional[torch.Tensor] = None,
               staging=None,
               prepared: Optional[PreparedEntries] = None) -> StepContext:
    """Lay out the step.  Every request must be admitted and its pages for this
    step reserved beforehand; nothing is committed here.

    The layout is a function of (tokens per entry, wanted rows per entry, width of
    the block tables) only.  ``min_pages`` widens the block tables, ``max_keys``
    overrides the context length used for planning, and ``into`` is a device
    buffer to fill instead of a new one: together they let a replayed HIP graph
    find every array at the address it was captured with.  ``staging`` is a pinned
    host buffer to lay the step out in, from which ``into`` is filled by a copy
    that does not block; the caller waits for that copy before it lays out the
    next step there; a ``StagingRing`` in its place hands out such buffers in turn and a new
    device buffer is filled from them.  ``prepared``: the same entries, already turned
    into arrays."""
    prep = prepared if prepared is not None else PreparedEntries(entries, cache, vocab_size)
    S = len(entries)
    counts, meta = prep.counts, prep.meta
    grans = np.asarray(sorted(set(int(g) for g in item_granularities)), dtype=np.int32)
    groups = cache.groups
    n_sections = 7 + 2 * len(groups) + 3 * len(grans)
    sections = np.zeros((2 * n_sections,), dtype=np.int64)
    ctx_arr, slot_arr = prep.ctx, prep.slots

    def call(out_ptr, cap):
        prep.build(cache, grans, max_position, min_pages, sections, out_ptr, cap)

    call(None, 0)                               # sizes first, then the buffer itself
    ring = staging if isinstance(staging, StagingRing) else None
    if ring is not None:
        staging = ring.take(int(meta[5]))
    if staging is not None:
        if staging.numel() < int(meta[5]) or staging.dtype != torch.int32:
            raise StepError(f"the step needs {int(meta[5])} int32 entries, the staging buffer "
                            f"holds {staging.numel()}")
        host = staging.numpy()[:int(meta[5])]
    else:
        host = np.empty((int(meta[5]),), dtype=np.int32)
    call(host.ctypes.data, host.size)
    T, R, max_pages = int(meta[0]), int(meta[2]), int(meta[3])
    names = ["token_ids", "positions", "token_seq", "seq_start", "ctx_len", "slot_id", "logit_rows"]
    for g in groups:
        names += [f"slots{g.index}", f"table{g.index}"]
    for gran in grans.tolist():
        names += [f"iseq{gran}", f"irow{gran}", f"icnt{gran}"]
    offsets = {name: (int(sections[2 * i]), int(sections[2 * i + 1])) for i, name in enumerate(names)}
    seq_lens, ctx_lens, slots = counts.tolist(), ctx_arr.tolist(), slot_arr.tolist()
    item_lists = {gran: offsets[f"iseq{gran}"][1] for gran in grans.tolist()}

    if into is None and ring is not None:
        dev = torch.empty((host.size,), dtype=torch.int32, device=device)
        dev.copy_(staging[:host.size], non_blocking=True)
        ring.copied()
    elif into is None:
        dev = torch.from_numpy(host).to(device)
    else:
        if into.numel() < host.size or into.dtype != torch.int32:
            raise StepError(f"the step needs {host.size} int32 entries, the buffer holds "
                            f"{into.numel()}")
        dev = into
        if staging is not None:
            dev[:host.size].copy_(staging[:host.size], non_blocking=True)
        else:
            dev[:host.size].copy_(torch.from_numpy(host))

    def view(name: str) -> torch.Tensor:
        off, n = offsets[name]
        return dev[off:off + n]

    ctx = StepContext(
        n_tokens=T, n_seqs=S, n_logit_rows=R,
        max_keys=max(max_keys, int(meta[4])),
        token_ids=view("token_ids"), positions=view("positions"), token_seq=view("token_seq"),
        seq_start=view("seq_start"), ctx_len=view("ctx_len"), slot_id=view("slot_id"),
        logit_rows=view("logit_rows"),
        seq_lens_host=seq_lens, ctx_lens_host=ctx_lens, slots_host=slots,
        host=host, offsets=offsets, table_width=max_pages)
    for g in groups:
        ctx.slot_mapping[g.index] = view(f"slots{g.index}")
        ctx.block_tables[g.index] = view(f"table{g.index}").view(S, max_pages)
    for gran, n_items in item_lists.items():
        ctx.items[gran] = (view(f"iseq{gran}"), view(f"irow{gran}"), view(f"icnt{gran}"), n_items)
    return ctx
