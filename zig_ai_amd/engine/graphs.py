"""Decode steps as HIP graphs.

A step in which every request brings exactly one token launches well over a
hundred small kernels; recorded once into a HIP graph and replayed, the step
costs one launch.  The reference does the same for its single sequence
(/root/reference/src/cuda/decode_graph.zig:44-143) and has to save and restore
the recurrent state around its capture (85-112) because its capture run also
executes; here the first step of a shape runs eagerly (so every kernel the shape
needs is loaded before anything is recorded) and recording executes nothing, so
no state is touched twice.

A graph is recorded per shape: number of requests, width of the block tables
(rounded up, so the table may grow inside the same graph) and the bucket of the
longest context (it fixes how the attention kernel cuts contexts).  Every
integer array of the step lives in one persistent device buffer that is
refilled before each replay, so the recorded kernels find their operands where
they were at capture.  Nothing in the graph clears memory with a memset node.
"""

from __future__ import annotations

import gc
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import raise_for
from ..kernels import host as hostlib
from .batch import PreparedEntries, StepEntry, StepError, build_step

PAGE_BUCKET = 64        # block-table width is rounded up to a multiple of this
KEYS_BUCKET = 1024      # and the longest context to a multiple of this
MAX_GRAPHS = 96         # recorded shapes kept; the one replayed longest ago goes first
MAX_PORTION_GRAPHS = 24 # the same for steps with prompt portions (their tensors are larger)
# A batch that a runner fills up with rows of its own (``ModelRunner.padding``) gets a
# recording without those rows once it has come this often as it is: recording costs about
# 2 ms, the rows some 0.01 ms each a step.
PROMOTE_AFTER = 64
# Steps with prompt portions are recorded only where the host is the limit (beyond some
# 1,000 tokens a step is bound by the GPU and a recording would only hold memory), and
# the recorded steps together hold at most this many bytes of intermediate tensors: the
# one replayed longest ago goes first.
PORTION_GRAPH_MAX_TOKENS = 1024
PORTION_GRAPH_BYTES = 2 << 30


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
        self.entries: Dict[Tuple[int, int, int], dict] = {}   # in order of last use
        self._arrays: Dict[int, dict] = {}       # per number of entries: arrays for the library
        self._lib = hostlib.lib()
        self.captures = 0
        self.replays = 0
        self._unpadded_sightings: Dict[Tuple[int, int, int], int] = {}
        # steps of any other shape (prompt portions, alone or beside single tokens)
        self.portion_entries: Dict[tuple, dict] = {}          # in order of last use
        self.portion_captures = 0
        self.portion_replays = 0

    def _scratch(self, S: int) -> dict:
        sc = self._arrays.get(S)
        if sc is None:
            sc = {"reqs": np.empty((S,), dtype=np.int64), "toks": np.empty((S,), dtype=np.int32),
                  "ones": np.ones((S,), dtype=np.int32), "zeros": np.zeros((S,), dtype=np.int32),
                  "ctx": np.empty((S,), dtype=np.int32), "slots": np.empty((S,), dtype=np.int32),
                  "meta": np.zeros((6,), dtype=np.int64), "extent": np.zeros((2,), dtype=np.int64)}
            sc["ptr"] = {k: v.ctypes.data for k, v in sc.items()}
            self._arrays[S] = sc
        return sc

    @staticmethod
    def _raise(rc: int, entries: Sequence[StepEntry]) -> None:
        if rc == hostlib.STEP:
            msg = hostlib.last_error()
            if msg.startswith("entry "):        # name the request instead of its place
                place = int(msg.split()[1].rstrip(":"))
                msg = f"request {entries[place].request!r}: " + msg.split(" ", 2)[2]
            raise StepError(msg)
        raise_for(rc)

    def run(self, runner, entries: Sequence[StepEntry],
            device_tokens: Optional[torch.Tensor] = None, more_to_come: bool = False,
            padded: bool = True) -> torch.Tensor:
        """Logits ``[len(entries), vocab]`` of a step of single tokens (one row per
        entry, whatever the entries want).  Takes the pages the new tokens need (all
        or none: ``OutOfPages`` leaves everything as it was).

        A shape's first step runs eagerly.  Recording costs about as much again and
        pays from the third step of the shape on, so the shape is recorded at once
        only when the caller says that ``more_to_come`` (it is about to issue further
        steps of the same requests); otherwise at its second step, which is then the
        graph's first replay.  While requests finish one after the other, every step
        has a batch size of its own that may never come back.

        With ``device_tokens`` (int32 ``[len(entries)]`` on the device, for instance
        what the sampler drew from the last step's logits) the entries' own tokens are
        ignored and the step reads its token ids from that tensor, copied on the
        device: the host never waits for them, so it can lay out this step while the
        last one is still running.

        A runner that pads its decode batches (``ModelRunner.padding``) adds rows of its
        own behind the entries of a batch that has no recording as it is (unless ``padded``
        is false); the step runs them like any request's, and their logits are not
        returned."""
        cache = runner.cache
        asked_for = len(entries)
        if device_tokens is not None and (device_tokens.dtype != torch.int32
                                          or device_tokens.numel() != asked_for):
            raise StepError(f"device_tokens must be int32 [{asked_for}]")
        lib = self._lib

        def prepare(entries):
            """The entries into the host library's arrays, their pages taken: the failure
            code (0: none), the arrays and the shape's key."""
            n = len(entries)
            sc = self._scratch(n)
            known = cache.handles.known
            reqs, toks = sc["reqs"], sc["toks"]
            for i, e in enumerate(entries):
                h = known(e.request)
                if h is None:
                    raise StepError(f"request {e.request!r} was not admitted")
                reqs[i] = h
                if device_tokens is not None:
                    toks[i] = 0                  # a stand-in; the ids are copied on the device
                    continue
                try:
                    toks[i] = e.tokens[0]
                except (OverflowError, TypeError, ValueError):
                    raise StepError(f"token id {e.tokens[0]!r} of request {e.request!r} is outside "
                                    f"the vocabulary of {self._vocab}") from None
            rc = lib.za_decode_prepare(cache.native, n, sc["ptr"]["reqs"], sc["ptr"]["toks"],
                                       self._vocab, self._max_position, sc["ptr"]["extent"])
            widest, longest = int(sc["extent"][0]), int(sc["extent"][1])
            return rc, sc, (n, _round_up(widest, PAGE_BUCKET), _round_up(longest, KEYS_BUCKET))

        rc, sc, key = prepare(entries)
        if rc == hostlib.OUT_OF_PAGES and padded and hasattr(runner, "release_padding") \
                and runner.release_padding():
            rc, sc, key = prepare(entries)       # with the pages that the runner's own rows held
        if rc:
            self._raise(rc, entries)
        pads = []
        recorded = self.entries.get(key)
        if padded and getattr(runner, "pad_decode", False) \
                and (recorded is None or recorded["graph"] is None):
            # The batch as it is has no recording.  Filled up to the next size that
            # recordings are kept for, it probably has; so that is what runs, until the batch
            # has come as it is PROMOTE_AFTER times: then it is worth a recording of its own,
            # which does not run the rows that fill it up.
            sightings = self._unpadded_sightings.get(key, 0) + 1
            if len(self._unpadded_sightings) > 4096:
                self._unpadded_sightings.clear()
            self._unpadded_sightings[key] = sightings
            if sightings <= PROMOTE_AFTER:
                pads = runner.padding(asked_for)
            if pads:
                filled = list(entries) + [StepEntry(name, [0], [0]) for name in pads]
                rc, sc_filled, key_filled = prepare(filled)
                if rc == hostlib.OUT_OF_PAGES:
                    # (cannot be: the rows hold their pages; but then the requests' own rows,
                    # whose pages are taken, run without them)
                    runner.release_padding()
                    pads = []
                elif rc:
                    self._raise(rc, filled)
                else:
                    entries, sc, key = filled, sc_filled, key_filled
        S = len(entries)
        ptr = sc["ptr"]
        slot = self.entries.get(key)
        if slot is not None:
            self.entries[key] = self.entries.pop(key)     # now the most recently used
        if slot is not None and slot["graph"] is not None:
            # Bring the persistent integer buffer up to date: the host library lays the
            # step out in the pinned staging buffer, and one copy that does not block
            # takes it to the device.  The layout equals the captured one because it
            # depends only on the number of entries and the table width.
            if slot["copied"] is not None:
                slot["copied"].synchronize()    # the last transfer out of the staging buffer
            pinned = slot["pinned"]
            rc = lib.za_step_build(cache.native, S, ptr["reqs"], ptr["ones"], ptr["toks"],
                                   ptr["ones"], ptr["zeros"], self._vocab, len(slot["grans"]),
                                   slot["grans_ptr"], self._max_position, key[1], slot["pinned_ptr"],
                                   slot["words"], slot["sections_ptr"], ptr["meta"], ptr["ctx"],
                                   ptr["slots"])
            if rc:
                self._raise(rc, entries)
            if int(sc["meta"][5]) != slot["words"]:
                raise StepError(f"the step's layout has {int(sc['meta'][5])} entries, the "
                                f"recorded one {slot['words']}")
            slot["buffer"].copy_(pinned, non_blocking=True)
            if slot["copied"] is None:
                slot["copied"] = torch.cuda.Event()
            slot["copied"].record()
            if device_tokens is not None:
                first = int(slot["sections"][0])          # where the token ids sit
                slot["buffer"][first:first + asked_for].copy_(device_tokens.view(-1))
            slot["graph"].replay()
            self.replays += 1
            return slot["logits"][:asked_for] if pads else slot["logits"]
        model = runner.model
        if device_tokens is not None:                     # a first step of this shape: on the host
            entries = [StepEntry(e.request, [t], [0])
                       for e, t in zip(entries, device_tokens.view(-1).tolist())] + list(entries[asked_for:])
        asked = [StepEntry(e.request, e.tokens, [0]) for e in entries]
        prepared = PreparedEntries(asked, cache, self._vocab)
        if slot is None:
            # size the persistent buffer with a dry layout on the host
            probe = build_step(asked, cache, torch.device("cpu"), self._vocab,
                               self._granularities, self._max_position,
                               min_pages=key[1], max_keys=key[2], prepared=prepared)
            words = probe.host.size
            grans = np.asarray(sorted(set(int(g) for g in self._granularities)), dtype=np.int32)
            slot = {"buffer": torch.full((words,), -1, dtype=torch.int32, device=runner.device),
                    "pinned": torch.empty((words,), dtype=torch.int32, pin_memory=True),
                    "graph": None, "logits": None, "copied": None, "words": words, "seen": 0,
                    "grans": grans,
                    "sections": np.zeros((2 * (7 + 2 * len(cache.groups) + 3 * len(grans)),),
                                         dtype=np.int64)}
            slot["grans_ptr"] = grans.ctypes.data
            slot["sections_ptr"] = slot["sections"].ctypes.data
            slot["pinned_ptr"] = slot["pinned"].data_ptr()
            # a graph holds its intermediate tensors for good: a process that sees many
            # batch sizes and context lengths keeps the shapes it used last
            if len(self.entries) >= MAX_GRAPHS:
                torch.cuda.current_stream().synchronize()    # its last replay may still run
                while len(self.entries) >= MAX_GRAPHS:
                    self.entries.pop(next(iter(self.entries)))
            self.entries[key] = slot
        ctx = build_step(asked, cache, runner.device, self._vocab, self._granularities,
                         self._max_position, min_pages=key[1], max_keys=key[2],
                         into=slot["buffer"], prepared=prepared)
        first = slot["seen"] == 0
        slot["seen"] += 1
        if first:
            logits = model.forward(ctx, runner.views)      # this step, eagerly
            if pads:
                logits = logits[:asked_for]
            if not more_to_come:
                return logits
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
        if first:
            return logits
        graph.replay()                                     # the shape's second step
        self.replays += 1
        return slot["logits"][:asked_for] if pads else slot["logits"]

    # ------------------------------------------------- steps with prompt portions
    def run_portions(self, runner, entries: Sequence[StepEntry]) -> torch.Tensor:
        """A step of any shape (pages already reserved): prompt portions, alone or beside
        single tokens.  A serving loop that cuts prompts into portions of one size issues
        the same shapes again and again (the reference's ``-ub 512``,
        /root/reference/src/main.zig:796-799), and a step of a few hundred tokens is some
        150 launches that the host issues more slowly than the GPU runs them; replayed
        from a graph the step is bound by the GPU again.

        The shape: tokens and wanted rows of every entry, in order, the width of the
        block tables and the longest context, both rounded up.  A shape's first step
        runs as it is; its second is recorded and replayed (so shapes that never come
        back cost nothing), every later one is a replay."""
        cache, model = runner.cache, runner.model
        prepared = PreparedEntries(entries, cache, self._vocab)
        if int(prepared.counts.sum()) > PORTION_GRAPH_MAX_TOKENS:
            ctx = build_step(entries, cache, runner.device, self._vocab, self._granularities,
                             self._max_position, prepared=prepared, staging=runner.staging)
            return model.forward(ctx, runner.views)
        grans = np.asarray(sorted(set(int(g) for g in self._granularities)), dtype=np.int32)
        sections = np.zeros((2 * (7 + 2 * len(cache.groups) + 3 * len(grans)),), dtype=np.int64)
        prepared.build(cache, grans, self._max_position, 0, sections, None, 0)     # sizes only
        widest, longest = int(prepared.meta[3]), int(prepared.meta[4])
        key = (tuple(prepared.counts.tolist()), tuple(prepared.want_counts.tolist()),
               _round_up(max(widest, 1), PAGE_BUCKET), _round_up(max(longest, 1), KEYS_BUCKET))
        slot = self.portion_entries.get(key)
        if slot is None:
            if len(self.portion_entries) >= 4 * MAX_PORTION_GRAPHS:    # sightings are cheap, not free
                for old in [k for k, v in self.portion_entries.items() if v["graph"] is None][:MAX_PORTION_GRAPHS]:
                    self.portion_entries.pop(old)
            self.portion_entries[key] = {"graph": None, "seen": 1, "bytes": 0}
            ctx = build_step(entries, cache, runner.device, self._vocab, self._granularities,
                             self._max_position, prepared=prepared, staging=runner.staging)
            return model.forward(ctx, runner.views)
        self.portion_entries[key] = self.portion_entries.pop(key)      # now the most recently used
        if slot["graph"] is None:
            probe = build_step(entries, cache, torch.device("cpu"), self._vocab, self._granularities,
                               self._max_position, min_pages=key[2], max_keys=key[3], prepared=prepared)
            words = probe.host.size
            recorded = [k for k, v in self.portion_entries.items() if v["graph"] is not None]
            held = sum(self.portion_entries[k]["bytes"] for k in recorded)
            while recorded and (len(recorded) >= MAX_PORTION_GRAPHS or held > PORTION_GRAPH_BYTES):
                torch.cuda.current_stream().synchronize()    # its last replay may still run
                held -= self.portion_entries.pop(recorded.pop(0))["bytes"]
            slot.update(buffer=torch.full((words,), -1, dtype=torch.int32, device=runner.device),
                        pinned=torch.empty((words,), dtype=torch.int32, pin_memory=True),
                        copied=None, words=words)
            ctx = build_step(entries, cache, runner.device, self._vocab, self._granularities,
                             self._max_position, min_pages=key[2], max_keys=key[3],
                             into=slot["buffer"], prepared=prepared)
            graph = torch.cuda.CUDAGraph()
            was_enabled = gc.isenabled()
            gc.disable()
            before = torch.cuda.memory_reserved(runner.device)
            try:
                with torch.cuda.graph(graph):                  # recorded, not executed
                    slot["logits"] = model.forward(ctx, runner.views)
            finally:
                if was_enabled:
                    gc.enable()
            slot["graph"] = graph
            # what the recording holds for good: its pool of intermediate tensors
            slot["bytes"] = max(0, torch.cuda.memory_reserved(runner.device) - before) + 8 * words
            self.portion_captures += 1
        else:
            if slot["copied"] is not None:
                slot["copied"].synchronize()        # the last transfer out of the staging buffer
            ctx = build_step(entries, cache, runner.device, self._vocab, self._granularities,
                             self._max_position, min_pages=key[2], max_keys=key[3],
                             into=slot["buffer"], staging=slot["pinned"], prepared=prepared)
            if ctx.host.size != slot["words"]:
                raise StepError(f"the step's layout has {ctx.host.size} entries, the recorded one "
                                f"{slot['words']}")
            if slot["copied"] is None:
                slot["copied"] = torch.cuda.Event()
            slot["copied"].record()
        slot["graph"].replay()
        self.portion_replays += 1
        return slot["logits"]
