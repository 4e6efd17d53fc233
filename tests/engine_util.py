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


class Forms:
    """Which of its equivalent forms each product of a bfloat16 run took, per request and
    position, read from the engine's own diagnostics (``ops.form_log``): a step of few
    tokens lets a projection run the norm before it, applies the SwiGLU gate to unrounded
    products and adds closing products to the stream unrounded; a step of many tokens
    rounds at each of these places.  ``rounding(i)`` turns request ``i``'s record into
    the ``plain.Rounding`` that makes the plain implementation round where the engine did.

    Steps replayed from a HIP graph leave no diagnostics; they took the forms of the step
    of the same shape (tokens, wanted rows) that was run before it was recorded."""

    def __init__(self, lengths, n_layers):
        import torch as _torch
        self.n_layers = n_layers
        self.flags = [dict() for _ in lengths]
        self.lengths = list(lengths)
        self.by_shape = {}
        self.kernels = set()
        self.seen = set()        # further forms a test may ask about (see note_step)
        self._torch = _torch

    def _mask(self, i, key):
        d = self.flags[i]
        if key not in d:
            d[key] = self._torch.zeros(self.lengths[i], dtype=self._torch.bool)
        return d[key]

    def note_step(self, entries, wanted_rows, log):
        """``entries``: (request, start, stop) of the step; ``log``: its records."""
        M = sum(b - a for _, a, b in entries)
        shape = (M, wanted_rows)
        products = [r for r in log if r["op"] in ("linear", "linear_swiglu")]
        for r in log:
            if r["op"] == "attention":
                self.kernels.add(r["kernel"])
            if r["op"] == "linear" and r.get("merged_ranges"):
                self.kernels.add("output projection that merges the ranges")
            if r["op"] == "attention_combine" or (r["op"] == "attention" and r.get("combine_kernel")):
                self.seen.add("ranges merged by the combine kernel")
            if r["op"] == "attention" and r["kernel"].startswith("decode_mfma") and r["rows"] > 16 \
                    and r["nsplit"] == 1:
                self.seen.add("decode attention of many rows, contexts uncut")
            if r["op"] == "linear" and r["M"] > 16 and r["partial_sums"] > 1:
                self.seen.add("library product with ranges of K")
            if r["op"] == "linear" and r.get("kernel") == "library" and r["added_to_stream"]:
                self.seen.add("library product added to the stream")
        if products:
            L = self.n_layers
            assert len(products) == 4 * L + (1 if wanted_rows else 0), \
                f"{len(products)} products in a step of a model with {L} layers"
            def wide(rec):
                import torch
                return bool(rec["added_to_stream"] or rec["partial_sums"] > 1
                            or rec["out"] == torch.float32)
            step = {}
            for l in range(L):
                m_in, m_out, gate, down = products[4 * l: 4 * l + 4]
                assert m_in["op"] == "linear" and m_out["op"] == "linear" and down["op"] == "linear"
                step[("late", (l, "mixer"))] = bool(m_in["norm_in_product"])
                step[("close", (l, "mixer"))] = wide(m_out)
                step[("late", (l, "feed_forward"))] = bool(gate["norm_in_product"])
                step[("gate", l)] = gate["op"] == "linear_swiglu"
                step[("close", (l, "feed_forward"))] = wide(down)
            step[("late", "head")] = bool(products[-1]["norm_in_product"]) if wanted_rows else False
            self.by_shape[shape] = step
        step = self.by_shape.get(shape)
        assert step is not None, f"a step of shape {shape} left no diagnostics and none ran before it"
        for i, a, b in entries:
            for key, value in step.items():
                if value:
                    self._mask(i, key)[a:b] = True

    def rounding(self, i):
        import plain_lfm2 as plain
        f = self.flags[i]
        gates = [f[k] for k in f if k[0] == "gate"]
        # (the gate's form is the same in every layer of a step: one mask)
        for g in gates[1:]:
            assert bool((g == gates[0]).all())
        return plain.Rounding(
            late_norm={k[1]: v for k, v in f.items() if k[0] == "late"},
            wide_gate=gates[0] if gates else None,
            wide_close={k[1]: v for k, v in f.items() if k[0] == "close"},
            probabilities=bool(self.kernels - {"plain"}))


def run_schedule(runner, prompts, schedule, wants=None, forms=None, streams=None):
    """Drive ``runner`` through ``schedule`` asking for the logits of every token (or, with
    ``wants``, of the positions ``wants[i]`` of request ``i``); returns one ``[wanted,
    vocab]`` tensor per request.  ``forms`` (a ``Forms``) collects how each step ran.
    ``streams`` (a dict) receives per request the residual stream after the embedding and
    after every layer, ``streams[i][layer] = [len, width]`` (such steps are not replayed
    from graphs)."""
    from zig_ai_amd.engine import StepEntry
    from zig_ai_amd.kernels import ops
    got = {i: [] for i in range(len(prompts))}
    for entries, ends in schedule:
        batch, counts = [], []
        for i, a, b in entries:
            if not runner.is_live(i):
                runner.admit(i)
            if wants is None:
                want = list(range(b - a))
            else:
                want = [p - a for p in wants[i] if a <= p < b]
            counts.append(len(want))
            batch.append(StepEntry(i, prompts[i][a:b], want))
        if forms is not None:
            ops.form_log = []
        taps = [] if streams is not None else None
        try:
            logits = (runner.step(batch, taps=taps) if taps is not None else runner.step(batch)).cpu()
        finally:
            log, ops.form_log = ops.form_log, None
        if taps is not None:
            row = 0
            for i, a, b in entries:
                per_layer = streams.setdefault(i, [dict() for _ in taps])
                for layer, named in enumerate(taps):
                    for name, t in named.items():
                        per_layer[layer].setdefault(name, []).append(t[row:row + (b - a)].cpu())
                row += b - a
        if forms is not None:
            forms.note_step(entries, sum(counts), log)
        row = 0
        for (i, a, b), n in zip(entries, counts):
            got[i].append(logits[row:row + n])
            row += n
        for i in ends:
            runner.release(i)
        runner.cache.check()
    if streams is not None:
        for i in list(streams):
            streams[i] = [{name: torch.cat(parts) if isinstance(parts, list) else parts
                           for name, parts in named.items()} for named in streams[i]]
    return [torch.cat(got[i]) if got[i] else torch.empty((0, 0)) for i in range(len(prompts))]


def layer_errors(oracle, prompt, taps, rounding, logits, rows=None):
    """Every layer of the plain implementation fed with what the engine fed its own:
    ``taps[l]["stream"]`` is the engine's residual stream before layer ``l`` (``[len,
    width]``, the whole request), and the plain layer's output is held against
    ``taps[l + 1]["stream"]``.  An attention layer is taken in three pieces, each fed
    what the engine had there: stream -> queries, keys, values (the keys and values as
    they lay in the cache); those -> the attention's output; that -> the rest of the
    block.  So every piece but the attention itself is a function of a token's own row.

    Returns ``[(what, worst row, median row)]``: a row's error is its largest deviation
    relative to the largest change the layer makes to the stream (for the embedding, the
    head and the attention's pieces: to the largest value).  An error made in one place
    shows there, undiluted by what follows and without what went before; a value that
    falls on the other side of a bfloat16 rounding boundary (the two sides sum in
    different orders) shows in its own row and not in the median."""
    n = len(prompt)
    dt = oracle.dtype
    out = []

    def rows_of(want, have, scale):
        assert torch.isfinite(have).all(), "non-finite values"
        want, have = want.reshape(want.shape[0], -1), have.reshape(have.shape[0], -1)
        e = (want - have).abs().max(dim=1).values / scale
        return float(e.max()), float(e.median())

    x0 = taps[0]["stream"].to(dt)
    out.append(("embedding",) + rows_of(oracle.embed(prompt), x0, x0.abs().max()))
    positions = torch.arange(n)
    n_layers = len(taps) - 1
    for l in range(n_layers):
        x = taps[l]["stream"].to(dt)
        after = taps[l + 1]
        name = f"layer {l} ({oracle.kinds[l]})"
        given = None
        if "o" in after:
            q, k, v = oracle.attention_qkv(l, x, positions, rounding)
            for what, want, have in (("queries", q, after["q"]), ("keys in the cache", k, after["k"]),
                                     ("values in the cache", v, after["v"])):
                out.append((f"{name}, {what}",) + rows_of(want, have.to(dt), want.abs().max()))
            import plain_lfm2 as plain
            o = plain.attention_output(after["q"].to(dt), after["k"].to(dt), after["v"].to(dt),
                                       positions, 0, rounding)
            given = after["o"].to(dt).reshape(n, -1)
            out.append((f"{name}, attention",) + rows_of(o, given, o.abs().max()))
            name += ", from the attention on"
        want = oracle.layer(l, x, positions, rounding, attention_output_given=given)
        change = (want - x).abs().max().clamp_min(1e-30)
        out.append((name,) + rows_of(want, after["stream"].to(dt), change))
    late = rounding.late_norm.get("head") if rounding is not None else None
    x = taps[n_layers]["stream"].to(dt)
    if rows is not None:
        idx = torch.as_tensor(list(rows), dtype=torch.long)
        x = x[idx]
        late = late[idx] if late is not None else None
    want = oracle.head(x, rounding, late)
    out.append(("head",) + rows_of(want, logits.to(dt), want.abs().max()))
    return out
