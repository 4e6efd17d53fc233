"""The Python entry point: ``Engine(model_dir).generate(prompts, ...)``.

The reference is driven from its command line only (/root/reference/src/main.zig:
573-1417: load, prefill in chunks, decode token by token, print); this class is
the same loop around the scheduler and the step function, for any number of
requests at once.
"""

from __future__ import annotations

import time
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..sampling.sampler import SamplingParams, sample_rows, uniforms
from ..cache.manager import CacheManager
from .batch import StepEntry
from .model import DecoderModel
from .runner import ModelRunner
from ..kernels import ops
from .scheduler import RUNNING, Request, ScheduledEntry, Scheduler


class Engine:
    def __init__(self, model_dir, dtype: str = "bfloat16", page_size: int = 16,
                 num_pages: Optional[int] = None, max_num_seqs: int = 64,
                 max_num_batched_tokens: int = 2048, chunk_size: int = 2048,
                 max_model_len: Optional[int] = None, use_graphs: bool = True,
                 portion_graphs: bool = False,
                 on_step=None, memory_fraction: float = 0.85, multi_step: int = 8,
                 reproducible: bool = False, warm_up: bool = True):
        """``model_dir``: a model folder, or a ``DecoderModel`` that is already built (from a
        folder or ``DecoderModel.from_random``; ``dtype`` and ``reproducible`` are then the
        model's own).
        ``num_pages``: pages per cache group; by default enough for
        ``max_num_seqs`` requests of ``max_model_len`` tokens (the model's
        ``max_position_embeddings`` if not given, capped at 8192), but no more than
        fit into ``memory_fraction`` of the device memory that is free once the
        weights are loaded.
        ``use_graphs=False`` launches every decode step kernel by kernel.
        ``portion_graphs=True`` also records steps with prompt portions, from the second
        time a shape is seen (see ``DecodeGraphs.run_portions``).
        ``multi_step``: while every running request decodes and none waits, up to this
        many decode steps are issued without the host waiting for the tokens in
        between (each step's tokens reach the next on the device), and the next such
        run is issued before the tokens of the last one are read; a request that
        meets its stop token inside a run wastes the steps issued after it, nothing
        else changes.  1 switches it off, and so does ``on_step``.
        ``on_step(info)``, if given, is called after every step with a dict:
        ``step``, ``plan`` (the scheduled entries), ``logits`` (32-bit, one row per
        entry that samples, on the device), ``tokens`` (what was drawn from them),
        ``seconds``.
        ``reproducible``: in bfloat16 the projections of a decode batch add to the residual
        stream with atomics, several ranges of K to one element in the hardware's order,
        so two runs agree to 32-bit rounding of the stream only; ``True`` keeps every sum
        in a fixed order (some 10 % slower decoding), and the same requests scheduled the
        same way then give the same bits.
        ``warm_up``: see ``Engine.warm_up``; done here, before the first request."""
        if isinstance(model_dir, DecoderModel):
            self.model = model_dir
        else:
            self.model = DecoderModel.from_folder(model_dir, dtype, reproducible=reproducible)
        limit = max_model_len or self.model.spec.max_position or 8192
        if max_model_len is None:
            limit = min(limit, 8192)
        if 0 < self.model.spec.max_position < limit:
            # positions beyond the model's own limit would stop a step in the middle of a
            # call of generate(), and every request of the call with it
            raise ValueError(f"max_model_len {limit} exceeds the model's max_position_embeddings "
                             f"{self.model.spec.max_position}")
        self.max_model_len = limit
        if num_pages is None:
            per_request = (limit + page_size - 1) // page_size
            num_pages = max_num_seqs * per_request
            per_page = CacheManager.bytes_per_page_index(self.model.cache_needs, page_size,
                                                         self.model.runtime.dtype)
            if per_page:
                free, _ = torch.cuda.mem_get_info(self.model.runtime.device)
                fit = int(free * memory_fraction) // per_page
                if fit < per_request:
                    raise MemoryError(
                        f"{free / 2**30:.1f} GiB of device memory are free: not enough for the "
                        f"cache of one request of {limit} tokens ({per_request * per_page / 2**30:.1f}"
                        " GiB); lower max_model_len")
                num_pages = min(num_pages, fit)
        # (the slots beyond max_num_seqs are for the rows that fill decode batches up to
        # recorded sizes, see ModelRunner.PAD_ROWS; they are given back when no request is left)
        self.runner = ModelRunner(self.model, page_size, num_pages,
                                  max_num_seqs + ModelRunner.PAD_ROWS - 1,
                                  use_graphs=use_graphs, portion_graphs=portion_graphs,
                                  pad_decode=use_graphs)
        self.on_step = on_step
        self.multi_step = 1 if on_step is not None else max(1, int(multi_step))
        self.scheduler = Scheduler(self.runner.cache, max_num_seqs, max_num_batched_tokens,
                                   chunk_size, limit)
        self._next_id = 0
        # (seconds_with_prompts: the part of step_seconds spent in steps that held prompt
        # portions; the rest went to steps of decoding requests only)
        self.timings = {"steps": 0, "step_seconds": 0.0, "seconds_with_prompts": 0.0,
                        "tokens_run": 0, "tokens_generated": 0}
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.max_num_seqs = int(max_num_seqs)
        self._token_staging = None       # pinned buffers for the tokens of runs of decode steps
        self._token_turn = 0
        self.warm_up_steps = self.warm_up() if warm_up else 0

    RUNS_PER_CALL = 8                 # runs of ``multi_step`` decode steps in one call of step()

    # ----------------------------------------------------------------- warm-up
    WARM_UP_MIN_WEIGHT = 1 << 19      # elements; smaller products are never timed

    def warm_up(self) -> int:
        """The GEMM library times its candidates for a shape at the shape's first call
        (10 to 60 ms a shape, shared by the row counts of a block, 17-32, 33-64, 65-128,
        129-255, then blocks of 256, where the library names a block's winner for them too).  Run one step of every block up to
        ``max_num_batched_tokens`` now, with a request of its own that is released again,
        so that no request pays for it (2.3 s at the 1.2B shape with a budget of 4,096 tokens,
        24 steps; 1.1 s at the 350M shape).  Nothing to do, and nothing done, for 32-bit
        models, models that take the library's first answer (``reproducible``,
        ZIG_AI_GEMM_TUNE=0) and models without a projection large enough to be timed.
        Returns the number of steps run."""
        from .model import walk_parts
        model, runner = self.model, self.runner
        rt = model.runtime
        wanted = ops.library_tuning if rt.tune is None else rt.tune
        if rt.dtype != torch.bfloat16 or not wanted:
            return 0
        top = [model.embedding, model.head] + [p for b in model.blocks for p in b.parts.values()]
        large = any(isinstance(v, torch.Tensor) and v.dim() == 2 and v.dtype == torch.bfloat16
                    and v.numel() >= self.WARM_UP_MIN_WEIGHT
                    for part in top for q in walk_parts(part) for v in vars(q).values())
        if not large:
            return 0
        # (up to 64 rows: the sizes that decode batches are filled up to; the heuristic does
        # not name the same algorithms for every row count of a block)
        sizes = [m for m in (24, 32, 40, 48, 56, 64, 128, 255) if m <= self.max_num_batched_tokens]
        sizes += list(range(256, self.max_num_batched_tokens + 1, 256))
        name = ("warm-up", id(self))
        steps = 0
        for m in sizes:
            if m > self.max_model_len:
                break
            # (steps of up to max_num_seqs rows want every row's logits, as a decode batch
            # of that many requests does: the head's shapes are met too)
            want = list(range(m)) if m <= max(self.max_num_seqs, 16) else [m - 1]
            runner.admit(name)
            try:
                if not runner.cache.can_reserve(name, m):
                    break
                runner.step([StepEntry(name, [0] * m, want)])
                steps += 1
            finally:
                runner.release(name)
        torch.cuda.synchronize(rt.device)
        return steps

    # ---------------------------------------------------------------- requests
    def add_request(self, prompt: Sequence[int], max_new_tokens: int,
                    sampling: Optional[SamplingParams] = None,
                    eos_token_id: Optional[int] = None, request_id: Hashable = None) -> Request:
        vocab = self.model.spec.vocab_size
        prompt = [int(t) for t in prompt]
        for t in prompt:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        if len(prompt) + max_new_tokens > self.max_model_len:
            raise ValueError(f"prompt of {len(prompt)} tokens plus {max_new_tokens} new ones "
                             f"exceeds max_model_len {self.max_model_len}")
        if request_id is None:
            request_id = self._next_id
            self._next_id += 1
        req = Request(request_id, prompt, max_new_tokens, sampling or SamplingParams(),
                      eos_token_id)
        self.scheduler.add(req)
        return req

    def step(self) -> List[Request]:
        """One scheduled step; returns the requests that finished in it."""
        plan = self.scheduler.schedule()
        if not plan:
            self.runner.release_padding()
            return []
        start = time.perf_counter()
        k = self._steps_ahead(plan)
        if k > 1:
            # (a call returns after at most RUNS_PER_CALL runs, so that a request added
            # between two calls waits no longer than that many steps)
            done = self._decode_many(plan, min(k, self.multi_step * self.RUNS_PER_CALL), start)
            if done and not self.scheduler.has_work():
                self.runner.release_padding()
            return done
        entries = []
        for e in plan:
            entries.append(StepEntry(e.request.id, e.request.span(e.start, e.count),
                                     [e.count - 1] if e.samples else []))
        logits = self.runner.step(entries)
        sampling = [e for e in plan if e.samples]
        drawn = sample_rows(
            logits, [e.request.sampling for e in sampling],
            uniforms([e.request.sampling.seed for e in sampling],
                     [e.request.number for e in sampling],
                     [len(e.request.output) for e in sampling]),
            [e.request.output for e in sampling])
        done = self.scheduler.update(plan, {e.request.id: t for e, t in zip(sampling, drawn)})
        self.timings["steps"] += 1
        elapsed = time.perf_counter() - start
        self.timings["step_seconds"] += elapsed
        if any(e.count > 1 or not e.samples or e.start == 0 for e in plan):
            self.timings["seconds_with_prompts"] += elapsed
        if self.on_step is not None:
            self.on_step({"step": self.timings["steps"] - 1, "plan": plan, "logits": logits,
                          "tokens": drawn, "seconds": elapsed})
        self.timings["tokens_run"] += sum(e.count for e in plan)
        self.timings["tokens_generated"] += len(sampling)
        if done and not self.scheduler.has_work():
            self.runner.release_padding()
        return done

    def _steps_ahead(self, plan: Sequence[ScheduledEntry]) -> int:
        """How many decode steps may follow this plan before the first of its requests
        reaches its length: more than one only if every entry is a decoding request,
        nobody waits to be admitted, and no request needs its history on the host
        between steps.  (``multi_step`` of them are issued in one go.)"""
        if self.multi_step <= 1 or self.scheduler.has_waiting():
            return 1
        k = 1 << 30
        for e in plan:
            req = e.request
            if e.count != 1 or not e.samples or e.start == 0 \
                    or req.sampling.repetition_penalty != 1.0:
                return 1
            k = min(k, req.max_new_tokens - len(req.output),
                    self.max_model_len - len(req.prompt) - len(req.output))
        return max(1, k)

    def _to_device(self, host: np.ndarray) -> torch.Tensor:
        """A small array to the device through pinned memory, without the host waiting
        (a copy from ordinary memory waits for everything issued before it)."""
        words = host.size
        ring = self.runner.staging
        pinned = ring.take(words)
        pinned.numpy()[:words] = host.view(np.int32)
        dev = torch.empty((words,), dtype=torch.int32, device=self.model.runtime.device)
        dev.copy_(pinned[:words], non_blocking=True)
        ring.copied()
        return dev

    def _decode_many(self, plan: Sequence[ScheduledEntry], horizon: int, start: float) -> List[Request]:
        """Decode steps of the plan's requests, ``multi_step`` at a time, until the first
        of them reaches its length (``horizon`` steps) or one meets its stop token.  The
        next run of steps is issued before the tokens of the last one are read, so the GPU
        does not wait while the host records them; a request that stops inside a run
        wastes the steps that were issued after its last token, nothing else."""
        reqs = [e.request for e in plan]
        ids = [r.id for r in reqs]
        params = [r.sampling for r in reqs]
        S = len(reqs)
        base = [len(r.output) for r in reqs]        # (the outputs grow only when tokens are read)
        greedy = all(p.greedy for p in params)
        if not greedy:
            fixed = self._to_device(np.concatenate([
                np.asarray([p.temperature for p in params], dtype=np.float32).view(np.int32),
                np.asarray([p.top_p for p in params], dtype=np.float32).view(np.int32),
                np.asarray([p.top_k for p in params], dtype=np.int32)]))
            temperature, top_p = fixed[:S].view(torch.float32), fixed[S:2 * S].view(torch.float32)
            top_k = fixed[2 * S:]
        if self._token_staging is None or self._token_staging[0].numel() < self.multi_step * S:
            self._token_staging = [torch.empty((self.multi_step * max(S, self.max_num_seqs),),
                                               dtype=torch.int32, pin_memory=True) for _ in range(3)]
        issued = 0
        in_flight: List[tuple] = []      # (first step, steps, pinned tokens, event), oldest first
        current: Optional[torch.Tensor] = None
        alive = list(range(S))
        done: List[Request] = []
        while True:
            n = min(self.multi_step, horizon - issued)
            more = n >= 1 and len(alive) == S and len(in_flight) < 2
            if more:
                if greedy:
                    def sample(logits: torch.Tensor, i: int) -> torch.Tensor:
                        return ops.argmax(logits)
                else:
                    u = self._to_device(np.asarray(
                        uniforms([p.seed for p in params] * n, [r.number for r in reqs] * n,
                                 [b + issued + i for i in range(n) for b in base]),
                        dtype=np.float32)).view(torch.float32).view(n, S)

                    def sample(logits: torch.Tensor, i: int, u=u) -> torch.Tensor:
                        return ops.sample(logits, temperature, top_k, top_p, u[i])
                tokens = [r.span(e.start, 1)[0] for r, e in zip(reqs, plan)] if current is None else None
                drawn = self.runner.decode_steps(ids, tokens, n, sample, device_tokens=current,
                                                 optional=current is not None)
                if drawn is None:                 # no pages for a further run
                    horizon = issued
                    continue
                steps = drawn.shape[0]
                pinned = self._token_staging[self._token_turn % 3]
                self._token_turn += 1
                pinned[:steps * S].copy_(drawn.view(-1), non_blocking=True)
                event = torch.cuda.Event()
                event.record()
                in_flight.append((issued, steps, pinned, event))
                issued += steps
                current = drawn[steps - 1]
                if steps < n:                     # pages ran out inside the run
                    horizon = issued
                if len(in_flight) < 2 and issued < horizon:
                    continue                      # the next run first, then this one's tokens
            if not in_flight:
                break
            first, steps, pinned, event = in_flight.pop(0)
            event.synchronize()                   # the one wait of the run
            rows = pinned[:steps * S].view(steps, S).tolist()
            for j, row in enumerate(rows):
                if not alive:
                    break
                step_plan = [ScheduledEntry(reqs[a], plan[a].start + first + j, 1, True) for a in alive]
                done += self.scheduler.update(step_plan, {reqs[a].id: row[a] for a in alive})
                self.timings["tokens_generated"] += len(alive)
                self.timings["tokens_run"] += len(alive)
                alive = [a for a in alive if reqs[a].phase == RUNNING]
            self.timings["steps"] += steps
        self.timings["step_seconds"] += time.perf_counter() - start
        return done

    def run(self) -> None:
        while self.scheduler.has_work():
            self.step()

    # ---------------------------------------------------------------- generate
    def generate(self, prompt_token_ids: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0,
                 repetition_penalty: float = 1.0, seed: int = 42,
                 eos_token_id: Optional[int] = None) -> List[List[int]]:
        """Generate for every prompt; returns the new tokens of each, in order.
        ``temperature <= 0`` is greedy.  Each request draws from its own random
        stream keyed by ``(seed, its number)``."""
        params = SamplingParams(temperature, top_k, top_p, repetition_penalty, seed)
        if eos_token_id is None:
            eos_token_id = getattr(getattr(self.model, "config", None), "eos_token_id", None)
        reqs: List[Request] = []
        try:
            for p in prompt_token_ids:
                reqs.append(self.add_request(p, max_new_tokens, params, eos_token_id))
            self.run()
        except BaseException:
            for r in reqs:                   # leave nothing of this call behind
                self.abort(r)
            raise
        return [list(r.output) for r in reqs]

    def abort(self, request: Request) -> None:
        """Take a request out of the engine; what it holds is given back."""
        self.scheduler.abort(request)
        if not self.scheduler.has_work():
            self.runner.release_padding()

    def stats(self) -> dict:
        out = self.runner.cache.stats()
        out.update(self.timings)
        out["preemptions"] = self.scheduler.preemption_count
        return out
