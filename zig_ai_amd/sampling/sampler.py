"""Choosing next tokens from the step's logits, on the device.

Options and their order follow the reference's sampler
(/root/reference/src/transformer/pipeline.zig:17-150): repetition penalty over the
tokens generated so far (main.zig:990, 1340 pass the generated tokens only, not
the prompt), temperature (<= 0 means greedy: the first index of the maximum),
top-k, top-p, then one draw per token.  Defaults are the reference's
(pipeline.zig:18-21, main.zig:34-39): temperature 1, top-k 0 (off), top-p 1 (off),
repetition penalty 1 (off), seed 42.

The reference draws from one generator shared by the whole run, which ties a
request's tokens to whatever ran beside it.  Here every request has its own
stream of uniform numbers, keyed by (seed, request number), one number per
generated token, so a request's tokens do not depend on batching, on the
scheduler's choices, or on being preempted and recomputed.
"""

from __future__ import annotations

from collections import Counter
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..kernels import host, ops


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    seed: int = 42

    def __post_init__(self):
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0 (0 switches it off)")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1] (1 switches it off)")
        if not self.repetition_penalty > 0.0:
            raise ValueError("repetition_penalty must be positive (1 switches it off)")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0


def uniforms(seeds: Sequence[int], request_numbers: Sequence[int],
             indices: Sequence[int]) -> List[float]:
    """Number ``indices[i]`` of the stream of ``(seeds[i], request_numbers[i])`` for
    every ``i``: 32-bit floats in [0, 1) from a counter-based generator in the host
    library (``csrc/host.cpp``), each a pure function of its three keys."""
    n = len(seeds)
    mask = 0xFFFFFFFFFFFFFFFF
    s = np.fromiter((int(v) & mask for v in seeds), dtype=np.uint64, count=n)
    r = np.fromiter((int(v) & mask for v in request_numbers), dtype=np.uint64, count=n)
    k = np.fromiter((int(v) & mask for v in indices), dtype=np.uint64, count=n)
    out = np.empty((max(n, 1),), dtype=np.float32)
    host.lib().za_uniforms(n, s.ctypes.data, r.ctypes.data, k.ctypes.data, out.ctypes.data)
    return out[:n].tolist()


class UniformStream:
    """The uniform numbers of one request: number ``k`` is a pure function of
    (seed, request number, k)."""

    def __init__(self, seed: int, request_number: int):
        self.seed = int(seed)
        self.request = int(request_number)

    def at(self, k: int) -> float:
        return uniforms([self.seed], [self.request], [k])[0]


def sample_rows(logits: torch.Tensor, params: Sequence[SamplingParams],
                uniforms: Sequence[float], histories: Sequence[Sequence[int]]) -> List[int]:
    """One token per row of ``logits [R, vocab]`` (32-bit, on the device)."""
    R = logits.shape[0]
    if not (len(params) == len(uniforms) == len(histories) == R):
        raise ValueError("one SamplingParams, uniform and history per row is needed")
    if R == 0:
        return []
    penalised = [r for r in range(R) if params[r].repetition_penalty != 1.0 and histories[r]]
    if penalised:
        rows, toks, facs = [], [], []
        for r in penalised:
            for tok, count in Counter(int(t) for t in histories[r]).items():
                rows.append(r)
                toks.append(tok)
                facs.append(params[r].repetition_penalty ** count)
        logits = logits.clone()
        dev = logits.device
        ops.repetition_penalty_(logits, torch.tensor(rows, dtype=torch.int32, device=dev),
                                torch.tensor(toks, dtype=torch.int32, device=dev),
                                torch.tensor(facs, dtype=torch.float32, device=dev))
    if all(p.greedy for p in params):
        return ops.argmax(logits).tolist()
    dev = logits.device
    packed = torch.tensor(
        [[p.temperature for p in params], [p.top_p for p in params], list(uniforms)],
        dtype=torch.float32).to(dev)
    top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32).to(dev)
    return ops.sample(logits, packed[0], top_k, packed[1], packed[2]).tolist()
