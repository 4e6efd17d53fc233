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

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence

from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages
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
    def __init__(self, cache: CacheManager, max_num_seqs: int = 64,
                 max_num_batched_tokens: int = 2048, chunk_size: int = 512,
                 max_model_len: int = 0):
        if max_num_batched_tokens < 1 or chunk_size < 1 or max_num_seqs < 1:
            raise ValueError("max_num_seqs, max_num_batched_tokens and chunk_size must be >= 1")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.chunk_size = chunk_size
        self.max_model_len = max_model_len
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self._arrivals = 0
        self.preemption_count = 0

    # ----------------------------------------------------------------- intake
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.id!r} has an empty prompt")
        if request.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        request.number = self._arrivals
        self._arrivals += 1
        request.phase = WAITING
        if request.max_new_tokens == 0:
            self._finish(request, "length")
            return
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # --------------------------------------------------------------- one step
    def schedule(self) -> List[ScheduledEntry]:
        budget = self.max_num_batched_tokens
        plan: List[ScheduledEntry] = []
        promised: Dict[int, int] = {}

        def fits(req: Request, n: int) -> bool:
            return self.cache.can_reserve(req.id, n, promised)

        def promise(req: Request, n: int) -> None:
            for gi, pages in self.cache.pages_needed(req.id, n).items():
                promised[gi] = promised.get(gi, 0) + pages

        # Decoding requests first (one token each), then running prompts, in arrival order.
        order = sorted(self.running, key=lambda r: (r.remaining != 1, r.number))
        for req in order:
            if req.phase != RUNNING:          # preempted while serving an earlier one
                continue
            if budget == 0:
                break
            n = min(req.remaining, budget, self.chunk_size)
            while not fits(req, n):
                victim = max((r for r in self.running if r.phase == RUNNING),
                             key=lambda r: r.number)
                if victim is req and len([r for r in self.running if r.phase == RUNNING]) == 1 \
                        and not plan:
                    raise OutOfPages(
                        f"request {req.id!r} needs more pages for {req.num_computed + n} tokens "
                        "than the whole pool holds")
                planned = next((e for e in plan if e.request is victim), None)
                if planned is not None:
                    # its pages for this step were only promised, not taken
                    for gi, pages in self.cache.pages_needed(victim.id, planned.count).items():
                        promised[gi] -= pages
                    budget += planned.count
                    plan.remove(planned)
                self._preempt(victim)
                if victim is req:
                    break
            if req.phase != RUNNING:
                continue
            promise(req, n)
            plan.append(ScheduledEntry(req, req.num_computed, n,
                                       req.num_computed + n == len(req.tokens)))
            budget -= n
        self.running = [r for r in self.running if r.phase == RUNNING]

        # Admit waiting requests, head of the line first, while everything fits.
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs \
                and self.cache.slots.free_count > 0:
            req = self.waiting[0]
            n = min(req.remaining, budget, self.chunk_size)
            self.cache.admit(req.id)
            if not fits(req, n):
                self.cache.release(req.id)
                if not self.running:
                    raise OutOfPages(
                        f"request {req.id!r} needs more pages for its first {n} tokens than "
                        "the whole pool holds")
                break
            self.waiting.popleft()
            req.phase = RUNNING
            self.running.append(req)
            promise(req, n)
            plan.append(ScheduledEntry(req, 0, n, n == len(req.tokens)))
            budget -= n
        return plan

    def _preempt(self, victim: Request) -> None:
        self.cache.release(victim.id)
        victim.num_computed = 0
        victim.phase = WAITING
        victim.preemptions += 1
        self.preemption_count += 1
        self.waiting.appendleft(victim)

    # ---------------------------------------------------------- after the step
    def update(self, plan: Sequence[ScheduledEntry], sampled: Dict[Hashable, int]) -> List[Request]:
        """Record the step: tokens computed, tokens drawn; finish and free what is done."""
        done = []
        for entry in plan:
            req = entry.request
            req.num_computed += entry.count
            if not entry.samples:
                continue
            token = int(sampled[req.id])
            req.output.append(token)
            if req.eos_token_id is not None and token == req.eos_token_id:
                self._finish(req, "eos")
            elif len(req.output) >= req.max_new_tokens:
                self._finish(req, "length")
            elif self.max_model_len and len(req.prompt) + len(req.output) >= self.max_model_len:
                self._finish(req, "max_model_len")
            if req.phase == FINISHED:
                done.append(req)
        self.running = [r for r in self.running if r.phase == RUNNING]
        return done

    def _finish(self, req: Request, reason: str) -> None:
        if req.id in self.cache.requests:
            self.cache.release(req.id)
        req.phase = FINISHED
        req.finish_reason = reason
        self.finished.append(req)
