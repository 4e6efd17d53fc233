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

from .batch import StepEntry, build_step

PAGE_BUCKET = 64        # block-table width is rounded up to a multiple of this
KEYS_BUCKET = 1024      # and the longest context to a multiple of this


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


class DecodeGraphs:
    """The recorded graphs of one runner.  It holds no reference to the runner: a
    cycle between the two would leave their destruction to the cyclic garbage
    collector, which may run at any allocation, also in the middle of a capture,
    and destroying another graph while a capture is open aborts the process."""

    def __init__(self):
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
        asked = [StepEntry(e.request, e.tokens, [0]) for e in entries]
        slot = self.entries.get(key)
        if slot is None:
            # size the persistent buffer with a dry layout on the host
            probe = build_step(asked, cache, torch.device("cpu"), model.spec.vocab_size,
                               model.item_granularities, model.spec.max_position,
                               min_pages=key[1], max_keys=key[2])
            words = probe.token_ids.untyped_storage().nbytes() // 4
            slot = {"buffer": torch.full((words,), -1, dtype=torch.int32, device=runner.device),
                    "graph": None, "logits": None}
            self.entries[key] = slot
        ctx = build_step(asked, cache, runner.device, model.spec.vocab_size,
                         model.item_granularities, model.spec.max_position,
                         min_pages=key[1], max_keys=key[2], into=slot["buffer"])
        if slot["graph"] is None:
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
        slot["graph"].replay()
        self.replays += 1
        return slot["logits"]
