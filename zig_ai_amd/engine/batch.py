"""The description of one step that the model's parts read: which tokens, whose
they are, where they sit in their requests, and where their cache lives.

A step packs the new tokens of all its requests into one row sequence
``[T]``: request 0's tokens, then request 1's, and so on.  A request contributes
a portion of its prompt (one token or many) or one decoded token; the model does
not distinguish the two.  Every integer array the kernels need is laid out in
ONE host buffer and copied to the device in one transfer.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import FREED, CacheManager


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


def build_step(entries: Sequence[StepEntry], cache: CacheManager, device: torch.device,
               vocab_size: int, item_granularities: Sequence[int] = (),
               max_position: int = 0, min_pages: int = 0, max_keys: int = 0,
               into: Optional[torch.Tensor] = None) -> StepContext:
    """Lay out the step.  Every request must be admitted and its pages for this
    step reserved beforehand; nothing is committed here.

    The layout is a function of (tokens per entry, wanted rows per entry, width of
    the block tables) only.  ``min_pages`` widens the block tables, ``max_keys``
    overrides the context length used for planning, and ``into`` is a device
    buffer to fill instead of a new one: together they let a replayed HIP graph
    find every array at the address it was captured with."""
    if not entries:
        raise StepError("a step needs at least one entry")
    seen = set()
    seq_lens, ctx_lens, slots = [], [], []
    for e in entries:
        if e.request in seen:
            raise StepError(f"request {e.request!r} appears twice in one step")
        seen.add(e.request)
        n = len(e.tokens)
        if n == 0:
            raise StepError(f"request {e.request!r} brings no tokens")
        for t in e.tokens:
            if not 0 <= int(t) < vocab_size:
                raise StepError(f"token id {t} of request {e.request!r} is outside the "
                                f"vocabulary of {vocab_size}")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise StepError(f"request {e.request!r} wants logits at place {w} of {n} tokens")
        ctx = cache.num_tokens(e.request)
        if max_position and ctx + n > max_position:
            raise StepError(f"request {e.request!r} would reach position {ctx + n - 1}, beyond "
                            f"max_position_embeddings {max_position}")
        seq_lens.append(n)
        ctx_lens.append(ctx)
        slots.append(cache.slot_of(e.request))
    T, S = sum(seq_lens), len(entries)
    R = sum(len(e.want) for e in entries)
    groups = cache.groups
    max_pages = 1
    for e in entries:
        for g in groups:
            max_pages = max(max_pages, len(cache.table(e.request, g.index)))
    max_pages = max(max_pages, min_pages)

    sections: List[Tuple[str, int]] = [
        ("token_ids", T), ("positions", T), ("token_seq", T), ("seq_start", S + 1),
        ("ctx_len", S), ("slot_id", S), ("logit_rows", R)]
    for g in groups:
        sections.append((f"slots{g.index}", T))
        sections.append((f"table{g.index}", S * max_pages))
    item_lists = {}
    for gran in sorted(set(item_granularities)):
        item_lists[gran] = _make_items(seq_lens, gran)
        w = len(item_lists[gran][0])
        sections += [(f"iseq{gran}", w), (f"irow{gran}", w), (f"icnt{gran}", w)]
    offsets, total = {}, 0
    for name, n in sections:
        offsets[name] = (total, n)
        total += (n + 3) // 4 * 4          # keep every section 16-byte aligned
    host = np.full((max(total, 4),), FREED, dtype=np.int32)

    def put(name: str, values) -> None:
        off, n = offsets[name]
        host[off:off + n] = values

    row = 0
    starts, logit_rows = [0], []
    for s, e in enumerate(entries):
        n = seq_lens[s]
        a, b = offsets["token_ids"][0] + row, offsets["token_ids"][0] + row + n
        host[a:b] = np.asarray(e.tokens, dtype=np.int32)
        a = offsets["positions"][0] + row
        host[a:a + n] = np.arange(ctx_lens[s], ctx_lens[s] + n, dtype=np.int32)
        a = offsets["token_seq"][0] + row
        host[a:a + n] = s
        logit_rows += [row + int(w) for w in e.want]
        for g in groups:
            a = offsets[f"slots{g.index}"][0] + row
            host[a:a + n] = cache.token_slots(e.request, g.index, ctx_lens[s], n)
            table = cache.table(e.request, g.index)
            a = offsets[f"table{g.index}"][0] + s * max_pages
            host[a:a + len(table)] = table
        row += n
        starts.append(row)
    put("seq_start", starts)
    put("ctx_len", ctx_lens)
    put("slot_id", slots)
    put("logit_rows", logit_rows)
    for gran, (seq, row0, cnt) in item_lists.items():
        put(f"iseq{gran}", seq)
        put(f"irow{gran}", row0)
        put(f"icnt{gran}", cnt)

    if into is None:
        dev = torch.from_numpy(host).to(device)
    else:
        if into.numel() < host.size or into.dtype != torch.int32:
            raise StepError(f"the step needs {host.size} int32 entries, the buffer holds "
                            f"{into.numel()}")
        dev = into
        dev[:host.size].copy_(torch.from_numpy(host))

    def view(name: str) -> torch.Tensor:
        off, n = offsets[name]
        return dev[off:off + n]

    ctx = StepContext(
        n_tokens=T, n_seqs=S, n_logit_rows=R,
        max_keys=max(max_keys, max(c + n for c, n in zip(ctx_lens, seq_lens))),
        token_ids=view("token_ids"), positions=view("positions"), token_seq=view("token_seq"),
        seq_start=view("seq_start"), ctx_len=view("ctx_len"), slot_id=view("slot_id"),
        logit_rows=view("logit_rows"),
        seq_lens_host=seq_lens, ctx_lens_host=ctx_lens, slots_host=slots,
        host=host, offsets=offsets, table_width=max_pages)
    for g in groups:
        ctx.slot_mapping[g.index] = view(f"slots{g.index}")
        ctx.block_tables[g.index] = view(f"table{g.index}").view(S, max_pages)
    for gran, (seq, _, _) in item_lists.items():
        ctx.items[gran] = (view(f"iseq{gran}"), view(f"irow{gran}"), view(f"icnt{gran}"), len(seq))
    return ctx
