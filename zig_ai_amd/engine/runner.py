"""The step function: a model, its cache, and ``step(entries) -> logits``.

One call runs exactly the tokens it is given, as one batch, from the cache that
earlier calls left, and returns the logits at the wanted places.  Generation
(through the scheduler) and trace replay both go through this class; there is
no second forward path.

The reference has no such function: its driver calls every layer for one
sequence, in chunks of ``--ubatch-size`` tokens and then token by token
(/root/reference/src/main.zig:795-865, 1138-1217), although its kernels are
written for several sequences (``num_seqs``, ``block_tables[seq]``:
/root/reference/src/cuda/paged_attention.cu:121-137).
"""

from __future__ import annotations

from typing import Callable, Hashable, List, Optional, Sequence

import torch

from ..cache.pages import OutOfPages, OutOfSlots
from .batch import StagingRing, StepContext, StepEntry, StepError, build_step
from .graphs import DecodeGraphs
from .model import DecoderModel


class ModelRunner:
    # A recorded decode step serves one number of requests.  With ``pad_decode`` a batch is
    # filled up to the next of 1, 2, 4, 8, 16 requests, beyond 16 to a multiple of PAD_ROWS,
    # with rows of the runner's own (each a request that stays at its first token), so that
    # batches which shrink or grow by a request at a time keep meeting recorded shapes.
    # (Up to 16 rows a step costs about the same at every size of 9 to 16 and of 1 to 8:
    # 0.69 ms at 1 request and 0.79 at 8 of the 1.2B shape; an unrecorded step costs 1.5.)
    # The rows are taken, and kept, only while every cache group has PAD_SPARE_PAGES free
    # pages and two for every request of the batch: in a pool that full the requests
    # themselves may need what the rows hold, and the scheduler counts it as taken.
    PAD_ROWS = 8
    PAD_SPARE_PAGES = 64

    @classmethod
    def padded_size(cls, n_requests: int) -> int:
        if n_requests <= 2:
            return n_requests
        if n_requests <= 16:
            return 1 << (n_requests - 1).bit_length()
        return -(-n_requests // cls.PAD_ROWS) * cls.PAD_ROWS

    def __init__(self, model: DecoderModel, page_size: int = 16, num_pages: int = 1024,
                 num_slots: int = 64, use_graphs: bool = True, portion_graphs: bool = False,
                 pad_decode: bool = False):
        """``use_graphs``: replay steps of single tokens as HIP graphs when every part
        of the model declares itself safe to record (``graph_safe``).  ``portion_graphs``:
        also steps with prompt portions, from the second time a shape is seen.
        ``pad_decode``: see ``PAD_ROWS``; the rows take up to ``PAD_ROWS - 1`` of the
        ``num_slots`` and a page each per cache group until ``release_padding``."""
        self.model = model
        self.device = model.runtime.device
        self.cache = model.make_cache(page_size, num_pages, num_slots)
        self.views = model.cache_views(self.cache)
        self.steps_run = 0
        # steps are laid out in pinned memory and copied without the host waiting
        self.staging = StagingRing() if self.device.type == "cuda" else None
        self.portion_graphs = bool(portion_graphs)
        self.graphs = (DecodeGraphs(model.spec.vocab_size, model.item_granularities, model.spec.max_position)
                       if (use_graphs and model.graph_safe) else None)

        self.pad_decode = bool(pad_decode) and self.graphs is not None
        self._pads: List[Hashable] = []

    # ------------------------------------------------------------- padding rows
    def padding(self, n_requests: int) -> List[Hashable]:
        """The requests that fill a decode batch of ``n_requests`` up to a recorded size:
        admitted, each with the pages of one token, which it never gets beyond.  Empty if
        the batch needs none, or if slots or pages for them cannot be had (then the rows
        that were there are given back too)."""
        if not self.pad_decode:
            return []
        rows = self.padded_size(n_requests) - n_requests
        if rows == 0:
            return []
        # (requests that decode in step need a page each at the same step)
        spare = max(self.PAD_SPARE_PAGES, 2 * n_requests) if self.PAD_SPARE_PAGES else 0
        if any(g.pool.free_count < spare for g in self.cache.groups):
            self.release_padding()
            return []
        try:
            while len(self._pads) < rows:
                name = ("padding row", id(self), len(self._pads))
                self.cache.admit(name)
                self._pads.append(name)
                self.cache.reserve(name, 1)
        except (OutOfPages, OutOfSlots):
            self.release_padding()
            return []
        return self._pads[:rows]

    def release_padding(self) -> int:
        """Give back what the padding rows hold; how many rows there were."""
        pads, self._pads = self._pads, []
        for name in pads:
            if name in self.cache.requests:
                self.cache.release(name)
        return len(pads)

    # ----------------------------------------------------------------- requests
    def admit(self, request: Hashable) -> None:
        self.cache.admit(request)

    def release(self, request: Hashable) -> None:
        self.cache.release(request)

    def is_live(self, request: Hashable) -> bool:
        return request in self.cache.requests

    # --------------------------------------------------------------------- step
    def reserve(self, entries: Sequence[StepEntry]) -> None:
        """Pages for every entry of the step, all of them or none."""
        try:
            self.cache.reserve_many([e.request for e in entries], [len(e.tokens) for e in entries])
        except KeyError as err:
            raise StepError(f"request {err.args[0]!r} was not admitted") from None

    def prepare(self, entries: Sequence[StepEntry]) -> StepContext:
        """Reserve pages for the entries and lay out the step."""
        self.reserve(entries)
        return build_step(entries, self.cache, self.device, self.model.spec.vocab_size,
                          self.model.item_granularities, self.model.spec.max_position,
                          staging=self.staging)

    def step(self, entries: Sequence[StepEntry],
             taps: Optional[list] = None) -> torch.Tensor:
        """Logits ``[R, vocab]`` (32-bit) at the wanted places, in the order of the
        entries and of each entry's ``want``.  ``taps``: see ``DecoderModel.forward``
        (such a step is never replayed from a graph)."""
        if taps is None and self.graphs is not None and entries \
                and all(len(e.tokens) == 1 for e in entries):
            logits = self._graph_step(entries)
        elif taps is None and self.graphs is not None and entries and self.portion_graphs:
            self.reserve(entries)
            logits = self.graphs.run_portions(self, entries)
        else:
            ctx = self.prepare(entries)
            logits = self.model.forward(ctx, self.views, taps)
        self.cache.commit_many([e.request for e in entries], [len(e.tokens) for e in entries])
        self.steps_run += 1
        return logits

    def decode_steps(self, requests: Sequence[Hashable], tokens: Optional[Sequence[int]], n_steps: int,
                     sample: Callable[[torch.Tensor, int], torch.Tensor],
                     device_tokens: Optional[torch.Tensor] = None,
                     optional: bool = False) -> Optional[torch.Tensor]:
        """Up to ``n_steps`` decode steps of the same requests without the host waiting
        in between: ``tokens`` are the requests' next tokens (or ``device_tokens``, int32
        ``[len(requests)]`` on the device, for instance the last tokens of an earlier
        call whose result the host has not read yet), ``sample(logits, i)`` draws the
        tokens of step ``i`` (int32 ``[len(requests)]`` on the device, without looking at
        them on the host), and those are the next step's tokens, handed over on the
        device.  Returns what was drawn, ``[steps done, len(requests)]`` on the device;
        fewer steps than asked for are done when pages run out after the first
        (``OutOfPages`` from the first step is raised, or with ``optional`` answered
        with ``None``: nothing was done)."""
        if device_tokens is None and (tokens is None or len(requests) != len(tokens)) or not requests:
            raise StepError("one next token per request is needed")
        if device_tokens is not None and (device_tokens.dtype != torch.int32
                                          or device_tokens.numel() != len(requests)):
            raise StepError(f"device_tokens must be int32 [{len(requests)}]")
        if device_tokens is not None and self.graphs is None:
            tokens = device_tokens.view(-1).tolist()
        entries = [StepEntry(r, [0 if tokens is None else t], [0])
                   for r, t in zip(requests, tokens if tokens is not None else requests)]
        ones = [1] * len(requests)
        drawn: List[torch.Tensor] = []
        current = device_tokens if self.graphs is not None else None
        for i in range(n_steps):
            try:
                if self.graphs is not None:
                    logits = self.graphs.run(self, entries, device_tokens=current,
                                             more_to_come=n_steps > 2)
                else:
                    if current is not None:
                        entries = [StepEntry(r, [t], [0])
                                   for r, t in zip(requests, current.view(-1).tolist())]
                    logits = self.model.forward(self.prepare(entries), self.views)
            except OutOfPages:
                if i == 0:
                    if optional:
                        return None
                    raise
                break
            current = sample(logits, i)
            drawn.append(current)
            self.cache.commit_many(requests, ones)
            self.steps_run += 1
        return torch.stack(drawn)

    def _graph_step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        for e in entries:
            for w in e.want:
                if int(w) != 0:
                    raise StepError(f"request {e.request!r} wants logits at place {w} of 1 token")
        logits = self.graphs.run(self, entries)
        rows = [i for i, e in enumerate(entries) for _ in e.want]
        if rows == list(range(len(entries))):
            return logits
        if not rows:
            return logits[:0]
        return logits.index_select(0, torch.tensor(rows, dtype=torch.long, device=logits.device))
