"""Decode steps as HIP graphs.

A step in which every request brings exactly one token launches well over a
hundred small kernels; recorded once into a HIP graph and replayed, the step
costs one launch.  The reference does the same for its single sequence
(/root/reference/src/cuda/decode_graph.zig:44-143) and has to save and restore
the recurrent state around its capture (85-112) because its capture run also
executes; here the first step of a shape runs eagerly (its results are the
step's results) and is then recorded without being executed, so no state is
touched twice.

A graph is recorded per shape: number of requests, width of the block tables
(rounded up, so the table may grow inside the same graph) and the bucket of the
longest context (it fixes how the attention kernel cuts contexts).  Every
integer array of the step lives in one persistent device buffer that is
refilled before each replay, so the recorded kernels find their operands where
they were at capture.  Nothing in the graph clears memory with a memset node.
"""

from __future__ import annotations

import gc
from typing import Dict, Sequence, Tuple

import torch

from .batch import StepEntry, StepError, build_step

PAGE_BUCKET = 64        # block-table width is rounded up to a multiple of this
KEYS_BUCKET = 1024      # and the longest context to a multiple of this


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


class DecodeGraphs:
    """The recorded graphs of one runner.  It holds no reference to the runner: a
    cycle between the two would leave their destruction to the cyclic garbage
    collector, which may run at any allocation, also in the middle of a capture,
    and destroying another graph while a capture is open aborts the process."""

    def __init__(self, vocab_size: int, item_granularities: Sequence[int], max_position: int):
        self._vocab = vocab_size
        self._granularities = tuple(item_granularities)
        self._max_position = max_position
        self.entries: Dict[Tuple[int, int, int], dict] = {}
        self.captures = 0
        self.replays = 0

    def run(self, runner, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits ``[len(entries), vocab]`` of a step of single tokens (one row per
        entry, whatever the entries want).  Pages must be reserved already."""
        cache, model = runner.cache, runner.model
        S = len(entries)
        widest = max((len(cache.table(e.request, g.index)) for e in entries for g in cache.groups),
                     default=1)
        longest = max(cache.num_tokens(e.request) + 1 for e in entries)
        key = (S, _round_up(widest, PAGE_BUCKET), _round_up(longest, KEYS_BUCKET))
        slot = self.entries.get(key)
        if slot is not None and slot["graph"] is not None:
            self._refill(slot, cache, entries, key)
            slot["graph"].replay()
            self.replays += 1
            return slot["logits"]
        asked = [StepEntry(e.request, e.tokens, [0]) for e in entries]
        if slot is None:
            # size the persistent buffer with a dry layout on the host
            probe = build_step(asked, cache, torch.device("cpu"), model.spec.vocab_size,
                               model.item_granularities, model.spec.max_position,
                               min_pages=key[1], max_keys=key[2])
            words = probe.host.size
            slot = {"buffer": torch.full((words,), -1, dtype=torch.int32, device=runner.device),
                    "pinned": torch.empty((words,), dtype=torch.int32, pin_memory=True),
                    "graph": None, "logits": None, "requests": None}
            self.entries[key] = slot
        ctx = build_step(asked, cache, runner.device, model.spec.vocab_size,
                         model.item_granularities, model.spec.max_position,
                         min_pages=key[1], max_keys=key[2], into=slot["buffer"])
        # keep the host image: later steps of the same requests only patch it
        slot["pinned"].numpy()[:] = ctx.host
        slot["offsets"] = ctx.offsets
        slot["requests"] = tuple(cache.serial_of(e.request) for e in entries)
        slot["table_lens"] = [[len(cache.table(e.request, g.index)) for g in cache.groups]
                              for e in entries]
        logits = model.forward(ctx, runner.views)          # this step, eagerly
        graph = torch.cuda.CUDAGraph()
        # No collection while the capture is open: a collector run could free
        # device memory or destroy an older graph, which a capture does not allow.
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):                  # recorded, not executed
                slot["logits"] = model.forward(ctx, runner.views)
        finally:
            if was_enabled:
                gc.enable()
        slot["graph"] = graph
        self.captures += 1
        return logits

    def _refill(self, slot: dict, cache, entries: Sequence[StepEntry], key) -> None:
        """Bring the persistent integer buffer up to date for this step.  When the
        step holds the same requests in the same order as the last one that used
        this graph, only what a decoded token changes is patched: token ids,
        positions, the new tokens' places, and block-table entries that were added."""
        if slot.get("copied") is not None:
            slot["copied"].synchronize()        # the last transfer out of the staging buffer
        host = slot["pinned"].numpy()
        off = slot["offsets"]
        admissions = tuple(cache.serial_of(e.request) for e in entries)
        requests = tuple(e.request for e in entries)
        S = len(entries)
        vocab = self._vocab
        for e in entries:
            t = int(e.tokens[0])
            if not 0 <= t < vocab:
                raise StepError(f"token id {t} of request {e.request!r} is outside the "
                                f"vocabulary of {vocab}")
        if admissions != slot["requests"]:
            asked = [StepEntry(e.request, e.tokens, [0]) for e in entries]
            fresh = build_step(asked, cache, torch.device("cpu"), vocab, self._granularities,
                               self._max_position, min_pages=key[1], max_keys=key[2])
            host[:] = fresh.host
            slot["requests"] = admissions
            slot["table_lens"] = [[len(cache.table(e.request, g.index)) for g in cache.groups]
                                  for e in entries]
        else:
            ctxs = [cache.num_tokens(r) for r in requests]
            if self._max_position and max(ctxs) + 1 > self._max_position:
                raise StepError(f"a request would reach position {max(ctxs)}, beyond "
                                f"max_position_embeddings {self._max_position}")
            a = off["token_ids"][0]
            host[a:a + S] = [int(e.tokens[0]) for e in entries]
            a = off["positions"][0]
            host[a:a + S] = ctxs
            a = off["ctx_len"][0]
            host[a:a + S] = ctxs
            ps = cache.page_size
            width = key[1]
            for gi, g in enumerate(cache.groups):
                sa = off[f"slots{g.index}"][0]
                ta = off[f"table{g.index}"][0]
                for s, r in enumerate(requests):
                    table = cache.table(r, g.index)
                    c = ctxs[s]
                    host[sa + s] = table[c // ps] * ps + c % ps
                    known = slot["table_lens"][s][gi]
                    if len(table) != known:
                        host[ta + s * width + known: ta + s * width + len(table)] = table[known:]
                        slot["table_lens"][s][gi] = len(table)
                    if g.need.window > 0:
                        # pages behind the window were given back: mark them
                        first = max(0, (c - g.need.window + 1) // ps)
                        if first:
                            host[ta + s * width: ta + s * width + first] = table[:first]
        slot["buffer"].copy_(slot["pinned"], non_blocking=True)
        if slot.get("copied") is None:
            slot["copied"] = torch.cuda.Event()
        slot["copied"].record()
