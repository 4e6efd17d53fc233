"""Helpers shared by the engine tests: model folders in a temporary place, and
ways of cutting the same requests into steps."""

import random
import tempfile

import torch

FOLDERS = {}


def model_folder(cfg: dict, seed: int, dtype=torch.float32, **kw) -> str:
    """A random model folder for ``cfg``, written once per process into a
    temporary directory (never into the repository)."""
    from zig_ai_amd.weights import write_random_model
    key = (repr(sorted(cfg.items())), seed, dtype, repr(sorted(kw.items())))
    if key not in FOLDERS:
        d = tempfile.mkdtemp(prefix="zigai_model_")
        write_random_model(cfg, d, seed=seed, dtype=dtype, **kw)
        FOLDERS[key] = d
    return FOLDERS[key]


def sharp_kwargs():
    """Weights under which faults show: attention scores spread over several
    units (so a lost or misplaced key changes the output), filters and norm
    weights that are not near-trivial."""
    return dict(std=0.05, norm_init="around_one",
                role_std={"norm": 0.3, "filter": 0.5, "bias": 0.1,
                          "q_proj.weight": 0.4, "k_proj.weight": 0.4})


def random_tokens(n: int, vocab: int, seed: int):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def rel_err(actual: torch.Tensor, expected: torch.Tensor) -> float:
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    assert a.shape == e.shape, (a.shape, e.shape)
    assert torch.isfinite(a).all(), "non-finite logits"
    return float((a - e).abs().max() / e.abs().max().clamp_min(1e-30))


# --- ways of cutting requests into steps ------------------------------------------------
# A schedule is a list of steps; a step is a list of (request index, start, stop) plus the
# list of requests that end after it.

def whole(lengths):
    """Each request alone, in one step."""
    return [([(i, 0, n)], [i]) for i, n in enumerate(lengths)]


def bulk_then_single(lengths, tail=32):
    """All but the last ``tail`` tokens in one step, then one token per step."""
    steps = []
    for i, n in enumerate(lengths):
        head = max(1, n - tail) if n > tail else 1
        steps.append(([(i, 0, head)], []))
        for p in range(head, n):
            steps.append(([(i, p, p + 1)], [i] if p == n - 1 else []))
        if head == n:
            steps[-1] = (steps[-1][0], [i])
    return steps


def changing_portions(lengths, seed=0, sizes=(16, 7, 2, 31, 3, 2, 1, 64, 5)):
    """Each request alone, in portions of changing size, down to two tokens (and one)."""
    steps = []
    k = seed
    for i, n in enumerate(lengths):
        p = 0
        while p < n:
            c = min(sizes[k % len(sizes)], n - p)
            k += 1
            steps.append(([(i, p, p + c)], [i] if p + c == n else []))
            p += c
    return steps


def mixed(lengths, seed=0, max_live=4, decode_tail=12):
    """Up to ``max_live`` requests at a time: each is fed in portions of random size
    until ``decode_tail`` tokens remain, then one token per step, so steps hold
    portions of some requests beside single tokens of others; a finished request
    makes room for the next.  Some requests sit out a step now and then."""
    rng = random.Random(seed)
    waiting = list(range(len(lengths)))
    live, cursor, steps = [], {}, []
    while waiting or live:
        while waiting and len(live) < max_live:
            i = waiting.pop(0)
            live.append(i)
            cursor[i] = 0
        entries, ends = [], []
        for i in list(live):
            n = lengths[i]
            if len(live) > 1 and rng.random() < 0.15:
                continue                                    # sits this step out
            left = n - cursor[i]
            if left <= decode_tail:
                c = 1
            else:
                c = min(left - decode_tail, rng.choice([2, 3, 5, 8, 13, 21, 40]))
            entries.append((i, cursor[i], cursor[i] + c))
            cursor[i] += c
            if cursor[i] == n:
                ends.append(i)
                live.remove(i)
        if entries:
            steps.append((entries, ends))
    return steps


def peak_tokens(lengths, schedule, round_to=64):
    """Most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held, peak = {}, 0
    for entries, ends in schedule:
        for i, a, b in entries:
            held[i] = b
        peak = max(peak, sum((v + round_to - 1) // round_to * round_to for v in held.values()))
        for i in ends:
            held.pop(i, None)
    return peak


def run_schedule(runner, prompts, schedule):
    """Drive ``runner`` through ``schedule`` asking for the logits of every token;
    returns one ``[len, vocab]`` tensor per request."""
    from zig_ai_amd.engine import StepEntry
    got = {i: [] for i in range(len(prompts))}
    for entries, ends in schedule:
        batch = []
        for i, a, b in entries:
            if not runner.is_live(i):
                runner.admit(i)
            batch.append(StepEntry(i, prompts[i][a:b], list(range(b - a))))
        logits = runner.step(batch).cpu()
        row = 0
        for i, a, b in entries:
            got[i].append(logits[row:row + (b - a)])
            row += b - a
        for i in ends:
            runner.release(i)
        runner.cache.check()
    return [torch.cat(got[i]) for i in range(len(prompts))]
