"""The scheduler: which requests run in the next step, and with how many tokens.

Kept from the reference's scheduler
(/root/reference/src/paged_attention/scheduler.zig:6-245): requests wait in
arrival order, are admitted while the cache has room (head of the line first,
97-134), decode until they reach ``max_new_tokens`` (236-245) and give their
pages back when they finish (221-234); when pages run out a running request is
preempted, the one that arrived last (156-168).

Different by design:
  * a token budget per step (``max_num_batched_tokens``, the reference's
    ``-b/--batch-size``) shared by decoding requests (one token each, served
    first) and by portions of prompts of at most ``chunk_size`` tokens (the
    reference's ``-ub/--ubatch-size``); the reference marks a whole prompt as
    processed in one go (141-145) and leaves the chunking to its driver;
  * pages are taken portion by portion, not for the whole prompt at admission
    (113-115);
  * preemption is by recomputation: the victim gives back all its pages and its
    state slot and returns to the FRONT of the waiting line with
    ``prompt + generated so far`` as the tokens to run again.  (The reference
    copies the victim's blocks to host memory, 170-191; here a request also
    carries convolution state, which recomputation restores exactly.)  A request
    is never preempted to admit a waiting one;
  * a request that cannot fit even alone raises ``OutOfPages`` instead of
    waiting forever.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages, raise_for  # noqa: F401  (OutOfPages: what schedule() raises)
from ..kernels import host as hostlib
from ..sampling.sampler import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    id: Hashable
    prompt: List[int]
    max_new_tokens: int
    sampling: SamplingParams = field(default_factory=SamplingParams)
    eos_token_id: Optional[int] = None
    number: int = 0                      # arrival number; also keys the request's random stream
    output: List[int] = field(default_factory=list)
    num_computed: int = 0                # tokens of prompt + output that are in the cache
    phase: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    def span(self, start: int, count: int) -> List[int]:
        """``tokens[start:start + count]`` without joining the two lists."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n:start - n + count]
        if start + count <= n:
            return self.prompt[start:start + count]
        return self.prompt[start:] + self.output[:start + count - n]

    @property
    def remaining(self) -> int:
        return len(self.prompt) + len(self.output) - self.num_computed


@dataclass
class ScheduledEntry:
    request: Request
    start: int          # first token (index into request.tokens) run in this step
    count: int
    samples: bool       # the step reaches the request's last token: a new token is drawn


class Scheduler:
    """The decisions are taken by the host library (``csrc/host.cpp``), which keeps
    each request's counters; this class keeps the ``Request`` objects (with their
    tokens) and mirrors the counters into them after every call."""

    _PHASES = (WAITING, RUNNING, FINISHED)
    _REASONS = (None, "eos", "length", "max_model_len")

    def __init__(self, cache: CacheManager, max_num_seqs: int = 64,
                 max_num_batched_tokens: int = 2048, chunk_size: int = 2048,
                 max_model_len: int = 0):
        if max_num_batched_tokens < 1 or chunk_size < 1 or max_num_seqs < 1:
            raise ValueError("max_num_seqs, max_num_batched_tokens and chunk_size must be >= 1")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.chunk_size = chunk_size
        self.max_model_len = max_model_len
        self._lib = hostlib.lib()
        self._ptr = self._lib.za_sched_new(cache.native, int(max_num_seqs),
                                           int(max_num_batched_tokens), int(chunk_size),
                                           int(max_model_len or 0))
        if not self._ptr:
            raise ValueError("the host library refused the scheduler's limits")
        self._requests: Dict[int, Request] = {}       # handle -> request, until forgotten
        self.finished: List[Request] = []
        cap = max(max_num_seqs, 1) + 1
        self._cap = cap
        self._ids = np.empty((cap,), dtype=np.int64)
        self._starts = np.empty((cap,), dtype=np.int32)
        self._counts = np.empty((cap,), dtype=np.int32)
        self._samples = np.empty((cap,), dtype=np.int32)
        self._tokens = np.empty((cap,), dtype=np.int32)
        self._victims = np.empty((cap,), dtype=np.int64)
        self._reasons = np.empty((cap,), dtype=np.int32)

    def __del__(self):
        ptr, self._ptr = getattr(self, "_ptr", None), None
        if ptr:
            self._lib.za_sched_free(ptr)

    # ----------------------------------------------------------------- intake
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.id!r} has an empty prompt")
        if request.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        handle = self.cache.pin(request.id)
        number = ctypes.c_longlong()
        eos = request.eos_token_id
        has_eos = eos is not None and -2 ** 31 <= int(eos) < 2 ** 31
        rc = self._lib.za_sched_add(self._ptr, handle, len(request.prompt),
                                    int(request.max_new_tokens), 1 if has_eos else 0,
                                    int(eos) if has_eos else 0, ctypes.byref(number))
        if rc:
            self.cache.unpin(request.id)
            raise_for(rc)
        request.number = number.value
        request.phase = WAITING
        self._requests[handle] = request
        if request.max_new_tokens == 0:
            self._finished(request, "length")

    def has_work(self) -> bool:
        return bool(self._lib.za_sched_has_work(self._ptr))

    def has_waiting(self) -> bool:
        return self._lib.za_sched_queue(self._ptr, 0, None, 0) > 0

    def _queue(self, which: int) -> List[Request]:
        n = self._lib.za_sched_queue(self._ptr, which, None, 0)
        out = np.empty((max(n, 1),), dtype=np.int64)
        self._lib.za_sched_queue(self._ptr, which, out.ctypes.data, n)
        return [self._requests[int(h)] for h in out[:n]]

    @property
    def waiting(self) -> List[Request]:
        return self._queue(0)

    @property
    def running(self) -> List[Request]:
        return self._queue(1)

    @property
    def preemption_count(self) -> int:
        return int(self._lib.za_sched_preemptions(self._ptr))

    # --------------------------------------------------------------- one step
    def schedule(self) -> List[ScheduledEntry]:
        n_plan, n_victims = ctypes.c_int(), ctypes.c_int()
        rc = self._lib.za_sched_schedule(
            self._ptr, self._cap, self._ids.ctypes.data, self._starts.ctypes.data,
            self._counts.ctypes.data, self._samples.ctypes.data, ctypes.byref(n_plan),
            self._victims.ctypes.data, ctypes.byref(n_victims))
        for h in self._victims[:min(n_victims.value, self._cap)].tolist():
            victim = self._requests[h]
            victim.num_computed = 0
            victim.phase = WAITING
            victim.preemptions += 1
        raise_for(rc)
        plan = []
        ids = self._ids[:n_plan.value].tolist()
        starts = self._starts[:n_plan.value].tolist()
        counts = self._counts[:n_plan.value].tolist()
        samples = self._samples[:n_plan.value].tolist()
        for h, start, count, sample in zip(ids, starts, counts, samples):
            req = self._requests[h]
            if req.phase != RUNNING:                  # admitted in this call
                req.phase = RUNNING
                self.cache.admitted_by_scheduler(req.id)
            plan.append(ScheduledEntry(req, start, count, bool(sample)))
        return plan

    # ---------------------------------------------------------- after the step
    def update(self, plan: Sequence[ScheduledEntry], sampled: Dict[Hashable, int]) -> List[Request]:
        """Record the step: tokens computed, tokens drawn; finish and free what is done."""
        n = len(plan)
        if n > self._cap:
            raise ValueError("a plan longer than max_num_seqs")
        handles = self.cache.handles
        for i, entry in enumerate(plan):
            req = entry.request
            self._ids[i] = handles.of(req.id)
            self._counts[i] = entry.count
            self._samples[i] = 1 if entry.samples else 0
            token = 0
            if entry.samples:
                token = int(sampled[req.id])
                req.output.append(token)
            self._tokens[i] = token
            req.num_computed += entry.count
        n_done = ctypes.c_int()
        raise_for(self._lib.za_sched_update(
            self._ptr, n, self._ids.ctypes.data, self._counts.ctypes.data,
            self._samples.ctypes.data, self._tokens.ctypes.data, self._victims.ctypes.data,
            self._reasons.ctypes.data, ctypes.byref(n_done)))
        done = []
        for h, reason in zip(self._victims[:n_done.value].tolist(),
                             self._reasons[:n_done.value].tolist()):
            req = self._requests[h]
            self._finished(req, self._REASONS[reason])
            done.append(req)
        return done

    def abort(self, req: Request) -> None:
        """Take a request out, waiting or running: its pages and slot are given back."""
        handle = self.cache.handles.known(req.id)
        if handle is None or handle not in self._requests:
            return                                   # finished already, or never added
        raise_for(self._lib.za_sched_abort(self._ptr, handle))
        req.phase = FINISHED
        req.finish_reason = "aborted"
        self._requests.pop(handle, None)
        self.cache.unpin(req.id)

    def _finished(self, req: Request, reason: str) -> None:
        handle = self.cache.handles.of(req.id)
        req.phase = FINISHED
        req.finish_reason = reason
        self.finished.append(req)
        self._lib.za_sched_forget(self._ptr, handle)
        self._requests.pop(handle, None)
        self.cache.unpin(req.id)
