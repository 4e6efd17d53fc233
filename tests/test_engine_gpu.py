"""The engine against the plain implementation, in 32-bit and in bfloat16, under
every way of cutting the work: whole requests; most of a request in one step and
the last 32 tokens one by one; portions of changing size; and mixed steps of up
to four live requests on so few pages that they are used again.

Bounds: each was measured first and then set with the margin stated beside it (the figures
in brackets are what was measured); none has been widened to let a run pass.

32-bit: logits within 1e-4 of the float64 plain implementation (relative to the request's
largest logit: accumulation order over a few layers), and every layer within 3e-5 of the
largest change it makes to the stream when the plain layer is fed what the engine fed its
own (measured 5e-6; a layer that changes the stream little is seen through the 32-bit
resolution of the stream itself).

bfloat16 has two bounds, because a bfloat16 run is chaotic at the level of single values:
the engine and the plain implementation add the same numbers up in different orders, a
sum that lies within 1e-7 of a rounding boundary of bfloat16 then falls on different sides
(measured: one value in 5,000 to 10,000), and that value is off by a whole 2^-8.

* Layer by layer (``check_layers``): the plain implementation computes in 32-bit, rounds to
  bfloat16 exactly where the engine does (``plain.Rounding``, from the engine's own record
  of the form each product took) and is fed, layer for layer, the stream the engine fed
  its own layer.  The MEDIAN row then agrees to 1e-4 (measured 1e-7 to 1.3e-5: most rows meet
  no such boundary inside one layer) and the WORST row to 8e-3 (measured 6e-3: a row that
  met one, seen against the layer's largest change to the stream).  This is the bound
  that can fail: a constant that is off by 1 % in a path only bfloat16 takes (the
  matrix-core attention's ``scale * log2(e)``, say) moves every row, the median with them,
  to 1e-3 and more.  Checked once with a build whose matrix-core attention kernels were
  given ``scale * log2(e) * 1.01``: every test of this file that runs them (configurations
  D, F, G and seven of the random ones, in every way of cutting) failed on the median, 2e-3
  to 8e-3 against the 1e-4 allowed, while the worst row alone would have passed half of
  them; with the scale changed by 0.3 % in the plain implementation the median still moves
  to 4e-4 and more.
* End to end against the float64 plain implementation: 4e-2 of the largest logit, which
  only says that nothing is grossly wrong.  About ten roundings of 2^-9 per layer; measured
  worst of 3,000 random configurations 2.6e-2 (five layers, width 1536, ``TINY_G`` below,
  kept as a case of its own), typical 1e-2.
"""


import pytest
import torch

import engine_util as eu
import plain_lfm2 as plain
from tiny_configs import REAL_2L, REAL_26B_2L, REAL_350M_2L, REAL_3L, TINY_A, TINY_B, TINY_C, TINY_D, TINY_E, TINY_F, TINY_G

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 4e-2}            # end to end, against float64
LAYER_WORST = {"float32": 3e-5, "bfloat16": 8e-3}    # layer by layer, the worst row
LAYER_MEDIAN = {"float32": 3e-5, "bfloat16": 1e-4}   # layer by layer, the median row
# At the real layer sizes every row of a bfloat16 run meets rounding boundaries (a row of the
# feed-forward holds 16,384 + 8,192 stored values, one in 5,000 of which falls on the other
# side), so there the median row is as far off as such a value moves it: measured up to
# 1.5e-3 of the layer's largest change.  What these sizes are run for are faults of
# indexing and dispatch at size (a tile's edge, a range of K, a split context), which are
# errors of order 1, not of a percent.
REAL_LAYER_MEDIAN = {"float32": 3e-5, "bfloat16": 4e-3}
# the same steps twice, replayed from a graph and not (contexts cut at other places: the
# order of 32-bit sums, and in bfloat16 the values that fall on a rounding boundary)
SAME_STEPS = {"float32": 2e-5, "bfloat16": 8e-3}
CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3), "F": (TINY_F, 5),
           "G": (TINY_G, 1029)}
LENGTHS = {"A": [5, 17, 33, 70], "B": [1, 8, 31, 64, 100], "C": [40, 3, 77], "D": [150, 9, 66, 40],
           "F": [130, 20, 75], "G": [130, 9]}
NAMES = ["A", "B", "C", "D", "F", "G"]

_cache = {}


def setup(name: str, dtype: str):
    """(model, float64 plain logits per request, prompts)."""
    key = (name, dtype)
    if key not in _cache:
        from zig_ai_amd.engine import DecoderModel
        cfg, seed = CONFIGS[name]
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = eu.model_folder(cfg, seed, store, **eu.sharp_kwargs())
        model = DecoderModel.from_folder(folder, dtype)
        oracle = plain.PlainLfm2(folder)
        prompts = [eu.random_tokens(n, cfg["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS[name])]
        expect = [oracle.logits(p) for p in prompts]
        # layer by layer: float64 for a 32-bit run; for a bfloat16 run the precision the
        # engine computes in, rounded where it rounds
        model.layer_oracle = oracle if dtype == "float32" else plain.PlainLfm2(folder, dtype=torch.float32)
        _cache[key] = (model, expect, prompts)
    return _cache[key]


def runner_for(model, page_size, num_pages, num_slots=4):
    from zig_ai_amd.engine import ModelRunner
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, num_slots=num_slots)


def check(got, expect, dtype, what):
    for i, (g, e) in enumerate(zip(got, expect)):
        err = eu.rel_err(g, e)
        assert err < TOL[dtype], f"{what}: request {i} off by {err:.3e} (allowed {TOL[dtype]:.1e})"


def check_layers(model, prompts, got, streams, forms, dtype, what, wants=None, median=LAYER_MEDIAN):
    """Every layer of every request against the plain layer fed the same stream."""
    for i, g in enumerate(got):
        rounding = forms.rounding(i) if dtype == "bfloat16" else None
        rows = wants[i] if wants is not None else None
        for part, worst, mid in eu.layer_errors(model.layer_oracle, prompts[i], streams[i],
                                                rounding, g, rows):
            allowed = LAYER_WORST[dtype]
            if "queries" in part or "keys" in part:
                # rotation angles are 32-bit products position * frequency: off by up to
                # 2 * 2^-24 of the angle, which is at most the position
                allowed += 1.2e-7 * len(prompts[i])
            assert worst < allowed and mid < median[dtype], \
                (f"{what}: request {i}, {part}: worst row off by {worst:.2e} (allowed "
                 f"{allowed:.1e}), median row by {mid:.2e} (allowed {median[dtype]:.0e})")


def run_and_check(model, runner, prompts, expect, schedule, dtype, what):
    """The schedule through the engine: logits against float64, every layer against the
    plain layer."""
    lengths = [len(p) for p in prompts]
    forms = eu.Forms(lengths, len(model.spec.layers))
    streams = {}
    got = eu.run_schedule(runner, prompts, schedule, forms=forms, streams=streams)
    check(got, expect, dtype, what)
    check_layers(model, prompts, got, streams, forms, dtype, what)
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_whole_requests(name, dtype):
    model, expect, prompts = setup(name, dtype)
    runner = runner_for(model, 16, 16)
    run_and_check(model, runner, prompts, expect, eu.whole(LENGTHS[name]), dtype, "whole")
    assert runner.cache.stats()["requests"] == 0
    assert all(g["pages_free"] == g["pages"] for g in runner.cache.stats()["groups"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_bulk_then_last_32_one_by_one(name, dtype):
    model, expect, prompts = setup(name, dtype)
    runner = runner_for(model, 4 if name == "A" else 8, 64)
    got = run_and_check(model, runner, prompts, expect, eu.bulk_then_single(LENGTHS[name], 32),
                        dtype, "bulk+tail")
    # and once more with the single tokens replayed from recorded graphs (no view into
    # the layers then): the same logits but for values on a rounding boundary
    replaying = runner_for(model, 4 if name == "A" else 8, 64)
    again = eu.run_schedule(replaying, prompts, eu.bulk_then_single(LENGTHS[name], 32))
    check(again, expect, dtype, "bulk+tail, replayed")
    assert replaying.graphs.replays >= 25
    # ... and the replayed steps are the steps issued kernel by kernel, to the bound of
    # two runs of the same steps (a recorded step plans its context ranges for a
    # rounded-up length, so some ranges are empty where the eager step has none)
    for i, (a, g) in enumerate(zip(again, got)):
        err = eu.rel_err(a, g.double())
        assert err < SAME_STEPS[dtype], f"request {i}: replayed and issued differ by {err:.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(name, dtype):
    model, expect, prompts = setup(name, dtype)
    for seed in (0, 3):
        runner = runner_for(model, 8 if name == "B" else 4, 64)
        run_and_check(model, runner, prompts, expect, eu.changing_portions(LENGTHS[name], seed),
                      dtype, f"portions seed {seed}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed_steps_with_page_reuse(name, dtype):
    model, expect, prompts = setup(name, dtype)
    # the same requests twice over, so that late ones land on pages early ones used
    lengths = LENGTHS[name] * 2
    prompts2, expect2 = prompts * 2, expect * 2
    page = 4
    for seed in (1, 2):
        schedule = eu.mixed(lengths, seed=seed, max_live=4 if seed == 1 else 3)
        pages = eu.peak_tokens(lengths, schedule, round_to=page) // page
        runner = runner_for(model, page, pages, num_slots=4)
        run_and_check(model, runner, prompts2, expect2, schedule, dtype, f"mixed seed {seed}")
        stats = runner.cache.stats()
        assert stats["pages_reused"] > 0, "the pool was too large to reuse a page"
        assert stats["slots_high_water"] <= 4


def test_cuts_agree_with_each_other():
    """The engine against itself in 32-bit: a different cut changes the order of a few
    sums only.  (In bfloat16 a step of few tokens rounds at other places than a step of
    many, so two cuts are each held against the plain implementation rounded their way:
    the tests above.)"""
    model, _, prompts = setup("B", "float32")
    a = eu.run_schedule(runner_for(model, 8, 64), prompts, eu.whole(LENGTHS["B"]))
    b = eu.run_schedule(runner_for(model, 8, 64), prompts, eu.changing_portions(LENGTHS["B"], 5))
    for x, y in zip(a, b):
        assert eu.rel_err(y, x.double()) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """300 tokens one by one after a short prompt: positions far beyond a page,
    a tile and a split of the attention kernel."""
    from zig_ai_amd.engine import StepEntry
    model, _, _ = setup("A", dtype)
    cfg, seed = CONFIGS["A"]
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, store, **eu.sharp_kwargs()))
    tokens = eu.random_tokens(7 + 300, cfg["vocab_size"], 55)
    expect = oracle.logits(tokens)
    runner = runner_for(model, 16, 32)
    runner.admit("r")
    got = [runner.step([StepEntry("r", tokens[:7], list(range(7)))]).cpu()]
    for p in range(7, len(tokens)):
        got.append(runner.step([StepEntry("r", tokens[p:p + 1], [0])]).cpu())
    assert eu.rel_err(torch.cat(got), expect) < TOL[dtype]
    # the single-token steps were replays of a recorded HIP graph ...
    assert runner.graphs is not None and runner.graphs.replays >= 290
    assert runner.graphs.captures <= 3
    # ... and replaying changes nothing but rounding (a recorded step cuts long
    # contexts at fixed places, an eager one by the step's own longest context)
    from zig_ai_amd.engine import ModelRunner
    eager = ModelRunner(model, page_size=16, num_pages=32, num_slots=4, use_graphs=False)
    eager.admit("r")
    again = [eager.step([StepEntry("r", tokens[:7], list(range(7)))]).cpu()]
    for p in range(7, len(tokens)):
        again.append(eager.step([StepEntry("r", tokens[p:p + 1], [0])]).cpu())
    assert eu.rel_err(torch.cat(again), torch.cat(got).double()) < SAME_STEPS[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("prompt_len,new", [(200, 120), (1000, 60)])
def test_graph_replay_across_shape_buckets(prompt_len, new, dtype):
    """A recorded decode step is kept per (requests, block-table width rounded up to 64
    pages, longest context rounded up to 1,024 keys).  With pages of 4 tokens a request
    decoded from 200 to 320 tokens crosses the table's bucket at 256, and one decoded from
    1,000 to 1,060 crosses both at 1,024: the step after the edge runs unrecorded, the next
    is recorded anew (another table width, another plan of context ranges, buffers of
    another size) and replayed.  Every step's logits against the plain implementation and
    against the same steps issued kernel by kernel."""
    from zig_ai_amd.engine import ModelRunner, StepEntry
    model, _, _ = setup("D", dtype)
    cfg, seed = CONFIGS["D"]
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, store, **eu.sharp_kwargs()))
    tokens = eu.random_tokens(prompt_len + new, cfg["vocab_size"], 77 + prompt_len)
    expect = oracle.logits(tokens, rows=list(range(prompt_len - 1, prompt_len + new)))
    pages = (prompt_len + new) // 4 + 2

    def run(use_graphs):
        runner = ModelRunner(model, page_size=4, num_pages=pages, num_slots=2, use_graphs=use_graphs)
        runner.admit("r")
        out = [runner.step([StepEntry("r", tokens[:prompt_len], [prompt_len - 1])]).cpu()]
        for p in range(prompt_len, prompt_len + new):
            out.append(runner.step([StepEntry("r", tokens[p:p + 1], [0])]).cpu())
            if p % 16 == 0:
                torch.cuda.synchronize()
        runner.release("r")
        runner.cache.check()
        return torch.cat(out), runner

    got, recorded = run(True)
    same, eager = run(False)
    assert eager.graphs is None
    assert recorded.graphs.captures >= 2, "the run stayed inside one recorded shape"
    assert recorded.graphs.replays >= new - 2 * recorded.graphs.captures - 1
    assert eu.rel_err(got, expect) < TOL[dtype]
    # step by step: the first step that differs names itself
    for k in range(got.shape[0]):
        err = eu.rel_err(got[k:k + 1], same[k:k + 1].double())
        assert err < SAME_STEPS[dtype], \
            f"position {prompt_len - 1 + k}: replayed and issued differ by {err:.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_between_other_work(dtype):
    """Replays of a recorded step interleaved with eager steps (portions of other
    requests), with synchronisations between them, each compared with the plain
    implementation; requests change slots and pages between replays."""
    from zig_ai_amd.engine import StepEntry
    model, expect, prompts = setup("B", dtype)
    runner = runner_for(model, 8, 64, num_slots=4)
    got = {i: [] for i in range(len(prompts))}
    # requests 3 and 4 (64 and 100 tokens) decode one token per step after a bulk
    # portion; requests 0..2 come and go between those steps
    for i, head in ((3, 30), (4, 50)):
        runner.admit(i)
        got[i].append(runner.step([StepEntry(i, prompts[i][:head], list(range(head)))]).cpu())
    cursor = {3: 30, 4: 50}
    others = [0, 1, 2, 0, 1, 2]
    step = 0
    while cursor[3] < 64 or cursor[4] < 100:
        batch = [StepEntry(i, prompts[i][cursor[i]:cursor[i] + 1], [0])
                 for i in (3, 4) if cursor[i] < len(prompts[i])]
        out = runner.step(batch).cpu()
        for row, e in enumerate(batch):
            got[e.request].append(out[row:row + 1])
            cursor[e.request] += 1
        torch.cuda.synchronize()
        if step % 5 == 0 and others:
            j = others.pop(0)
            runner.admit(("x", j))
            o = runner.step([StepEntry(("x", j), prompts[j], list(range(len(prompts[j]))))]).cpu()
            assert eu.rel_err(o, expect[j]) < TOL[dtype]
            runner.release(("x", j))
        step += 1
    for i in (3, 4):
        assert eu.rel_err(torch.cat(got[i]), expect[i]) < TOL[dtype]
    assert runner.graphs.replays >= 40


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_portions_replayed_from_graphs(dtype):
    """Prompts cut into portions of one size, as a serving loop cuts them: from the second
    time a shape is seen the step is recorded, then replayed, also beside decoded tokens of
    another request and with other requests' steps and synchronisations between the
    replays.  Every replay gives what the same step gives when it is issued kernel by
    kernel, and both give the plain implementation's logits."""
    from zig_ai_amd.engine import ModelRunner
    model, expect, prompts = setup("D", dtype)          # 150, 9, 66 and 40 tokens
    lengths = LENGTHS["D"]
    schedule = []
    for i, n in enumerate(lengths):                      # each alone, 32 tokens at a time
        for a in range(0, n, 32):
            schedule.append(([(i, a, min(n, a + 32))], [i] if a + 32 >= n else []))
    # and two together: portions of 32 of one beside single tokens of the other
    both = [([(0, 0, 32), (2, 0, 32)], [])]
    for k in range(1, 4):
        both.append(([(0, 32 * k, 32 * k + 32), (2, 31 + k, 32 + k)], []))
    both.append(([(0, 128, 150), (2, 35, 66)], [0, 2]))
    recorded = ModelRunner(model, page_size=8, num_pages=64, num_slots=4, portion_graphs=True)
    eager = ModelRunner(model, page_size=8, num_pages=64, num_slots=4)
    for sched, which in ((schedule, range(4)), (both, (0, 2)), (schedule, range(4))):
        got = eu.run_schedule(recorded, prompts, sched)
        same = eu.run_schedule(eager, prompts, sched)
        for i in which:
            assert eu.rel_err(got[i], expect[i]) < TOL[dtype]
            assert eu.rel_err(got[i], same[i].double()) < SAME_STEPS[dtype]
        torch.cuda.synchronize()
    g = recorded.graphs
    assert g.portion_captures >= 3 and g.portion_replays >= 12
    assert eager.graphs.portion_replays == 0
    recorded.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(dtype):
    """The very first positions: one token alone, two, three (shorter than the
    convolution), each as its own request."""
    model, _, _ = setup("B", dtype)
    cfg, seed = CONFIGS["B"]
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, store, **eu.sharp_kwargs()))
    prompts = [[7], [7, 300], [9, 9, 9], [511, 0, 1, 2]]
    lengths = [len(p) for p in prompts]
    expect = [oracle.logits(p) for p in prompts]
    got = eu.run_schedule(runner_for(model, 8, 8), prompts, eu.whole(lengths))
    check(got, expect, dtype, "first tokens")
    got = eu.run_schedule(runner_for(model, 8, 8), prompts,
                          eu.changing_portions(lengths, 0, sizes=(1,)))
    check(got, expect, dtype, "first tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wanted_rows_only(dtype):
    """Logits come back only for the wanted places, in the order asked."""
    from zig_ai_amd.engine import StepEntry
    model, expect, prompts = setup("A", dtype)
    runner = runner_for(model, 4, 64)
    for i in (1, 2):
        runner.admit(i)
    out = runner.step([StepEntry(1, prompts[1], [16, 0]), StepEntry(2, prompts[2], []),
                       ]).cpu()
    assert out.shape == (2, TINY_A["vocab_size"])
    assert eu.rel_err(out, expect[1][[16, 0]]) < TOL[dtype]
    none = runner.step([StepEntry(1, [3], [])])
    assert none.shape == (0, TINY_A["vocab_size"])


def test_step_errors():
    from zig_ai_amd.cache import OutOfPages
    from zig_ai_amd.engine import StepEntry, StepError
    model, _, prompts = setup("A", "float32")
    runner = runner_for(model, 4, 4)
    runner.admit("a")
    with pytest.raises(StepError, match="vocabulary"):
        runner.step([StepEntry("a", [256], [0])])
    with pytest.raises(StepError, match="not admitted"):
        runner.step([StepEntry("b", [1], [0])])
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", list(range(17)), [0])])
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes(dtype):
    """Two layers (ShortConv, attention) at the sizes of the LFM2-1.2B shape, vocabulary
    65,536: whole, in portions with single tokens, and batched with another request."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = eu.model_folder(REAL_2L, 7, store, std=0.02, norm_init="around_one",
                             role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                       "k_proj.weight": 0.05})
    model = DecoderModel.from_folder(folder, dtype)
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 65536, 900 + n) for n in (40, 21)]
    expect = [oracle.logits(p) for p in prompts]
    runner = ModelRunner(model, page_size=16, num_pages=16, num_slots=2)
    got = eu.run_schedule(runner, prompts, eu.whole([40, 21]))
    check(got, expect, dtype, "whole")
    schedule = [([(0, 0, 20)], []), ([(0, 20, 21), (1, 0, 17)], []), ([(0, 21, 22), (1, 17, 18)], []),
                ([(0, 22, 38), (1, 18, 19)], []), ([(0, 38, 39), (1, 19, 20)], []),
                ([(0, 39, 40), (1, 20, 21)], [0, 1])]
    got = eu.run_schedule(runner, prompts, schedule)
    check(got, expect, dtype, "portions beside single tokens")


REAL_LENGTHS = [760, 300, 130, 260]
_real = {}


def real_setup(dtype):
    if dtype not in _real:
        from zig_ai_amd.engine import DecoderModel
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = eu.model_folder(REAL_3L, 7, store, std=0.02, norm_init="around_one",
                                 role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                           "k_proj.weight": 0.05})
        model = DecoderModel.from_folder(folder, dtype)
        oracle = plain.PlainLfm2(folder)
        model.layer_oracle = oracle if dtype == "float32" else plain.PlainLfm2(folder, dtype=torch.float32)
        prompts = [eu.random_tokens(n, 65536, 900 + n) for n in REAL_LENGTHS]
        # the head (65,536 rows of 2,048) at some forty places per request: spread over
        # the request, and its last eight
        wants = [sorted(set(range(0, n, max(1, n // 30))) | set(range(n - 8, n))) for n in REAL_LENGTHS]
        expect = [oracle.logits(p, rows=w) for p, w in zip(prompts, wants)]
        _real[dtype] = (model, prompts, wants, expect)
    return _real[dtype]


def real_schedule(kind):
    n = REAL_LENGTHS
    if kind == "whole":                      # 760 rows in one step: beyond every small-batch form
        return eu.whole(n)
    if kind == "bulk":                       # decoding at contexts beyond 640: cut contexts, merged
        return eu.bulk_then_single(n, 32)
    if kind == "portions":
        return eu.changing_portions(n, 0)
    if kind == "far portion":                # 128 tokens that start 620 tokens into their request
        return [([(0, 0, 620)], []), ([(0, 620, 748), (1, 0, 300)], [1]), ([(0, 748, 760)], [0]),
                ([(2, 0, 130), (3, 0, 3)], [2]), ([(3, 3, 260)], [3])]
    return eu.mixed(n, seed=4, max_live=3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["whole", "bulk", "portions", "mixed", "far portion"])
def test_real_layer_sizes_every_way_of_cutting(kind, dtype):
    """Three layers (ShortConv, attention, ShortConv) at the LFM2-1.2B shape's sizes, with a
    vocabulary of 65,536, requests of 760, 300, 130 and 260 tokens: the forms that only such
    sizes take (library products of hundreds of rows with and without ranges of K, the
    decode kernels that run the norm and add to the stream, attention work items of 128
    rows over a dozen key tiles, contexts cut into ranges and merged), as a model and layer
    by layer, against the plain implementation."""
    from zig_ai_amd.engine import ModelRunner
    model, prompts, wants, expect = real_setup(dtype)
    schedule = real_schedule(kind)
    pages = eu.peak_tokens(REAL_LENGTHS, schedule, round_to=16) // 16
    runner = ModelRunner(model, page_size=16, num_pages=pages, num_slots=3)
    forms = eu.Forms(REAL_LENGTHS, 3)
    streams = {}
    got = eu.run_schedule(runner, prompts, schedule, wants=wants, forms=forms, streams=streams)
    check(got, expect, dtype, kind)
    check_layers(model, prompts, got, streams, forms, dtype, kind, wants=wants, median=REAL_LAYER_MEDIAN)
    stats = runner.cache.stats()
    assert stats["requests"] == 0 and stats["slots_high_water"] <= 3
    if kind == "mixed":
        assert stats["pages_reused"] > 0, "the pool was too large to reuse a page"
    if dtype == "bfloat16":
        kernels = forms.kernels
        assert "mfma" in kernels and ("decode_mfma_rope" in kernels or kind in ("whole", "far portion"))
        if kind == "bulk":        # single tokens of one request, its context cut into ranges
            assert "output projection that merges the ranges" in kernels


LONG_TOKENS, LONG_BULK, SHORT_REQUESTS = 2100, 2068, 23
_long = {}


def long_context_setup(dtype):
    """Two layers at the 1.2B shape's sizes; one request of 2,100 tokens and 23 short ones."""
    if dtype not in _long:
        from zig_ai_amd.engine import DecoderModel
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = eu.model_folder(REAL_2L, 7, store, std=0.02, norm_init="around_one",
                                 role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                           "k_proj.weight": 0.05})
        model = DecoderModel.from_folder(folder, dtype)
        oracle = plain.PlainLfm2(folder)
        model.layer_oracle = oracle if dtype == "float32" else plain.PlainLfm2(folder, dtype=torch.float32)
        # request 0 is the long one; 1..7 decode 32 tokens beside it, 8..23 the last 16
        heads = [LONG_BULK] + [4 + (5 * r) % 9 for r in range(1, SHORT_REQUESTS + 1)]
        lengths = [LONG_TOKENS] + [heads[r] + (32 if r <= 7 else 16) for r in range(1, SHORT_REQUESTS + 1)]
        prompts = [eu.random_tokens(n, 65536, 2000 + r) for r, n in enumerate(lengths)]
        wants = [sorted(set(range(0, LONG_BULK, 103)) | {2070, 2075, 2083} | set(range(2092, 2100)))]
        wants += [[n - 2, n - 1] for n in lengths[1:]]
        expect = [oracle.logits(p, rows=w) for p, w in zip(prompts, wants)]
        schedule = [([(0, 0, LONG_BULK)], []),
                    ([(r, 0, heads[r]) for r in range(1, SHORT_REQUESTS + 1)], [])]
        for k in range(32):
            live = range(0, 8) if k < 16 else range(0, SHORT_REQUESTS + 1)
            at = lambda r: heads[r] + (k if r <= 7 else k - 16)
            schedule.append(([(r, at(r), at(r) + 1) for r in live],
                             list(range(SHORT_REQUESTS + 1)) if k == 31 else []))
        _long[dtype] = (model, prompts, lengths, wants, expect, schedule)
    return _long[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_at_a_context_beyond_2048_at_real_layer_sizes(dtype):
    """The decode steps that the throughput figures are taken from, as a model: a request of
    2,100 tokens decoded one by one, sixteen steps beside 7 short requests (a step of 8
    rows: the long context cut into ranges of 512 keys, ranges that are empty for the short
    requests, merged by the combine kernel) and sixteen beside 23 (24 rows: library
    products, K in ranges where N is small, attention uncut), against the plain
    implementation, layer by layer; then the same steps once more, replayed from recorded
    graphs, against the plain logits and against the first run."""
    from zig_ai_amd.engine import ModelRunner
    model, prompts, lengths, wants, expect, schedule = long_context_setup(dtype)
    pages = eu.peak_tokens(lengths, schedule, round_to=16) // 16
    runner = ModelRunner(model, page_size=16, num_pages=pages, num_slots=SHORT_REQUESTS + 1)
    forms = eu.Forms(lengths, 2)
    streams = {}
    got = eu.run_schedule(runner, prompts, schedule, wants=wants, forms=forms, streams=streams)
    check(got, expect, dtype, "issued")
    check_layers(model, prompts, got, streams, forms, dtype, "issued", wants=wants,
                 median=REAL_LAYER_MEDIAN)
    if dtype == "bfloat16":
        assert "decode_mfma_rope" in forms.kernels
        assert "ranges merged by the combine kernel" in forms.seen
        assert "decode attention of many rows, contexts uncut" in forms.seen
        assert "library product with ranges of K" in forms.seen
        # (the long request's first step, more than 1,024 rows: w2 added to the stream by
        # the library itself)
        assert "library product added to the stream" in forms.seen
    replaying = ModelRunner(model, page_size=16, num_pages=pages, num_slots=SHORT_REQUESTS + 1)
    again = eu.run_schedule(replaying, prompts, schedule, wants=wants)
    assert replaying.graphs.captures >= 2 and replaying.graphs.replays >= 24
    check(again, expect, dtype, "replayed")
    for i, (a, g) in enumerate(zip(again, got)):
        err = eu.rel_err(a, g.double())
        assert err < SAME_STEPS[dtype], f"request {i}: replayed and issued differ by {err:.2e}"


OTHER_SHAPES = {"350m": REAL_350M_2L, "2.6b": REAL_26B_2L}
OTHER_LENGTHS = [200, 60, 130]
_other = {}


def other_shape_setup(shape, dtype):
    if (shape, dtype) not in _other:
        from zig_ai_amd.engine import DecoderModel
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = eu.model_folder(OTHER_SHAPES[shape], 11, store, std=0.02, norm_init="around_one",
                                 role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                           "k_proj.weight": 0.05})
        model = DecoderModel.from_folder(folder, dtype)
        oracle = plain.PlainLfm2(folder)
        model.layer_oracle = oracle if dtype == "float32" else plain.PlainLfm2(folder, dtype=torch.float32)
        prompts = [eu.random_tokens(n, 65536, 3000 + n) for n in OTHER_LENGTHS]
        wants = [sorted(set(range(0, n, max(1, n // 10))) | set(range(n - 4, n))) for n in OTHER_LENGTHS]
        expect = [oracle.logits(p, rows=w) for p, w in zip(prompts, wants)]
        _other[(shape, dtype)] = (model, prompts, wants, expect)
    return _other[(shape, dtype)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["whole", "bulk", "mixed"])
@pytest.mark.parametrize("shape", ["350m", "2.6b"])
def test_layer_sizes_of_the_other_measured_shapes(shape, kind, dtype):
    """Two layers (ShortConv, attention) at the sizes the 350M shape has (hidden 1,024, 16
    query heads on 8 key/value heads, feed-forward 4,608) and at the 2.6B shape's feed-forward
    width (7,168), requests of 200, 60 and 130 tokens: whole, most of a request and then its
    last 32 tokens one by one, and mixed on few pages; as a model and layer by layer."""
    from zig_ai_amd.engine import ModelRunner
    model, prompts, wants, expect = other_shape_setup(shape, dtype)
    assert model.config.intermediate_size == (4608 if shape == "350m" else 7168)
    n = OTHER_LENGTHS
    schedule = {"whole": eu.whole(n), "bulk": eu.bulk_then_single(n, 32),
                "mixed": eu.mixed(n, seed=6, max_live=3)}[kind]
    pages = eu.peak_tokens(n, schedule, round_to=16) // 16
    runner = ModelRunner(model, page_size=16, num_pages=pages, num_slots=3)
    forms = eu.Forms(n, 2)
    streams = {}
    got = eu.run_schedule(runner, prompts, schedule, wants=wants, forms=forms, streams=streams)
    check(got, expect, dtype, f"{shape} {kind}")
    check_layers(model, prompts, got, streams, forms, dtype, f"{shape} {kind}", wants=wants,
                 median=REAL_LAYER_MEDIAN)
    assert runner.cache.stats()["requests"] == 0
    if kind == "bulk":        # and the single tokens once more, replayed from graphs
        replaying = ModelRunner(model, page_size=16, num_pages=pages, num_slots=3)
        again = eu.run_schedule(replaying, prompts, schedule, wants=wants)
        assert replaying.graphs.replays >= 60
        check(again, expect, dtype, f"{shape} {kind}, replayed")
        for i, (a, g) in enumerate(zip(again, got)):
            assert eu.rel_err(a, g.double()) < SAME_STEPS[dtype], f"request {i}"


def test_reproducible_decoding_at_real_layer_sizes():
    """With ``reproducible`` two runs of the same steps give the same bits in bfloat16
    (no atomic additions to the stream: the norms add the stacks of partial sums up in
    their order); without it they agree within the tolerance, and both agree with the
    plain implementation."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    folder = eu.model_folder(REAL_2L, 7, torch.bfloat16, std=0.02, norm_init="around_one",
                             role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                       "k_proj.weight": 0.05})
    prompts = [eu.random_tokens(n, 65536, 950 + n) for n in (24, 9, 17)]
    oracle = plain.PlainLfm2(folder)
    expect = [oracle.logits(p) for p in prompts]

    def run(reproducible):
        model = DecoderModel.from_folder(folder, "bfloat16", reproducible=reproducible)
        assert model.runtime.stream_additions == (not reproducible)
        runner = ModelRunner(model, page_size=16, num_pages=12, num_slots=3)
        # the first tokens as one portion each, the rest as decode steps of three requests
        schedule = [([(0, 0, 5), (1, 0, 5), (2, 0, 5)], [])]
        for t in range(5, 24):
            live = [(r, t, t + 1) for r, n in enumerate((24, 9, 17)) if t < n]
            schedule.append((live, [r for r, n in enumerate((24, 9, 17)) if t == n - 1]))
        return eu.run_schedule(runner, prompts, schedule)

    first, second = run(True), run(True)
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    check(first, expect, "bfloat16", "reproducible")
    check(run(False), expect, "bfloat16", "with additions to the stream")


def test_a_decode_step_at_real_layer_sizes_runs_no_norm_kernel(monkeypatch):
    """What the fused forms are for: in a bfloat16 step of a few tokens every norm runs
    inside the projection that follows it and every mixer and feed-forward adds to the
    stream itself, so the norm kernel and the stacks of partial sums do not appear; in a
    step of many tokens, and with ``reproducible``, they do."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    from zig_ai_amd.kernels import ops
    folder = eu.model_folder(REAL_2L, 7, torch.bfloat16, std=0.02, norm_init="around_one")
    calls = {"norm": 0, "stacks": 0}
    norm_kernel, linear = ops.add_rmsnorm, ops.linear

    def counting_norm(*a, **kw):
        calls["norm"] += 1
        return norm_kernel(*a, **kw)

    def counting_linear(*a, **kw):
        y = linear(*a, **kw)
        if y is not None and y.dim() == 3:
            calls["stacks"] += 1
        return y

    monkeypatch.setattr(ops, "add_rmsnorm", counting_norm)
    monkeypatch.setattr(ops, "linear", counting_linear)
    for reproducible in (False, True):
        model = DecoderModel.from_folder(folder, "bfloat16", reproducible=reproducible)
        runner = ModelRunner(model, page_size=16, num_pages=8, num_slots=2, use_graphs=False)
        runner.admit("a")
        runner.admit("b")
        for tokens, few in (([list(range(30)), list(range(30, 52))], False), ([[5], [6]], True),
                            ([list(range(50, 62)), list(range(70, 80))], "some")):
            calls.update(norm=0, stacks=0)
            runner.step([StepEntry("a", tokens[0], [len(tokens[0]) - 1]),
                         StepEntry("b", tokens[1], [len(tokens[1]) - 1])])
            if few is True and not reproducible:
                assert calls == {"norm": 0, "stacks": 0}, calls
            elif few == "some" and not reproducible:
                # 22 rows: the mixers' closing products add themselves to the stream and the
                # feed-forwards' first products run their norms (one kernel for norm, gate|up
                # and gate); the mixers' norms (which add w2's stacks) and the final one stay
                assert calls == {"norm": 3, "stacks": 2}, calls
            else:
                # two layers: four norms and the final one (the first is handed over and
                # run by the projection's binding, which this count does not see);
                # out_proj / w2 leave stacks
                assert calls["norm"] >= 4 and calls["stacks"] >= 2, calls


def test_graph_replays_with_library_products():
    """Decode batches beyond 16 rows send their projections to the GEMM library (K in
    ranges as a batched product where N is small, 32-bit logits): such steps are
    recorded too.  Every replay, with eager work and synchronisations between the
    replays, must give what the same step gives unrecorded."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    folder = eu.model_folder(REAL_2L, 7, torch.bfloat16, std=0.02, norm_init="around_one",
                             role_std={"norm": 0.2, "filter": 0.5, "q_proj.weight": 0.05,
                                       "k_proj.weight": 0.05})
    model = DecoderModel.from_folder(folder, "bfloat16")
    B = 24
    prompts = [eu.random_tokens(5 + r % 7, 65536, 700 + r) for r in range(B)]
    tails = [eu.random_tokens(8, 65536, 800 + r) for r in range(B)]
    runners = [ModelRunner(model, page_size=16, num_pages=3 * B, num_slots=B + 1, use_graphs=g)
               for g in (True, False)]
    for runner in runners:
        for r in range(B):
            runner.admit(r)
        runner.step([StepEntry(r, prompts[r], []) for r in range(B)])
    extra = eu.random_tokens(30, 65536, 999)
    for step in range(8):
        batch = [StepEntry(r, [tails[r][step]], [0]) for r in range(B)]
        recorded, eager = (runner.step(batch).cpu() for runner in runners)
        # the recorded step plans its attention for a rounded-up context length, so
        # the two may differ as two cuts of the same work do: in rounding
        assert eu.rel_err(recorded, eager.double()) < SAME_STEPS["bfloat16"], f"step {step}"
        if step % 2 == 1:                     # other work between the replays
            for runner in runners:
                runner.admit(("x", step))
                runner.step([StepEntry(("x", step), extra, [29])])
                runner.release(("x", step))
        torch.cuda.synchronize()
    assert runners[0].graphs.replays >= 6 and runners[1].graphs is None
    oracle = plain.PlainLfm2(folder)                     # and the last replay is right
    for r in (0, 12, 23):
        want = oracle.logits(prompts[r] + tails[r])[-1:]
        assert eu.rel_err(recorded[r:r + 1], want) < TOL["bfloat16"], f"request {r}"


def test_widths_that_are_no_multiple_of_eight():
    """Any width runs in 32-bit; bfloat16 projections need rows that start on 16-byte
    boundaries and say so when the model is built, before anything runs."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    from zig_ai_amd.kernels import KernelError
    folder = eu.model_folder(TINY_E, 4, torch.float32, **eu.sharp_kwargs())
    model = DecoderModel.from_folder(folder, "float32")
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 131, 40 + n) for n in (37, 6)]
    expect = [oracle.logits(p) for p in prompts]
    got = eu.run_schedule(ModelRunner(model, 4, 32, 2), prompts, eu.changing_portions([37, 6], 2))
    check(got, expect, "float32", "odd widths")
    narrow = eu.model_folder(TINY_E, 4, torch.bfloat16, **eu.sharp_kwargs())
    with pytest.raises(KernelError, match="multiple of 8"):
        DecoderModel.from_folder(narrow, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_hand_tokens_over_on_the_device(dtype):
    """Several decode steps without the host reading the tokens in between: the same
    tokens as step by step, including across the first step of a new graph shape and
    when pages run out in the middle."""
    from zig_ai_amd.engine import StepEntry
    from zig_ai_amd.kernels import ops
    model, _, prompts = setup("B", dtype)
    long_prompt = max(prompts, key=len)
    greedy = lambda logits, i: ops.argmax(logits)
    ids = ["a", "b", "c"]
    lens = [9, 30, 17]

    def start(runner):
        last = []
        for r, n in zip(ids, lens):
            runner.admit(r)
            logits = runner.step([StepEntry(r, long_prompt[:n], [n - 1])])
            last.append(int(ops.argmax(logits)[0]))
        return last

    single = runner_for(model, 8, 64)
    cur = start(single)
    want = []
    for _ in range(20):
        logits = single.step([StepEntry(r, [t], [0]) for r, t in zip(ids, cur)])
        cur = ops.argmax(logits).tolist()
        want.append(cur)
    many = runner_for(model, 8, 64)
    cur = start(many)
    got = []
    for k in (1, 7, 12):                                  # 12: crosses a page and a graph shape
        drawn = many.decode_steps(ids, cur, k, greedy)
        assert drawn.shape == (k, 3) and drawn.dtype == torch.int32
        got += drawn.tolist()
        cur = got[-1]
    if dtype == "float32":
        assert got == want
    else:
        assert sum(g != w for g, w in zip(got, want)) <= 1   # a near-tie may tip in bfloat16
    # a pool that holds the prompts and little more: the run stops when pages run out
    tight = runner_for(model, 8, 9)                       # 2 + 4 + 3 pages for the prompts
    cur = start(tight)
    drawn = tight.decode_steps(ids, cur, 16, greedy)
    assert 1 <= drawn.shape[0] < 16
    tight.cache.check()
    assert [tight.cache.num_tokens(r) for r in ids] == [n + drawn.shape[0] for n in lens]
    if dtype == "float32":
        assert drawn.tolist() == want[:drawn.shape[0]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_batches_with_padding_rows(dtype):
    """A decode batch of 19 requests filled up to 24 with rows of the runner's own: every
    request's logits are those of the plain implementation at each step (run as it is,
    recorded, replayed), the batch of 17 that is left when two requests end meets the same
    recording, and a runner without slots to spare records the batch as it is."""
    from zig_ai_amd.engine import ModelRunner, StepEntry
    model, _, _ = setup("D", dtype)
    cfg, seed = CONFIGS["D"]
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, store, **eu.sharp_kwargs()))
    ids = list(range(19))
    lens = [3 + (7 * i) % 23 for i in ids]
    new = 5
    seqs = [eu.random_tokens(n + new, cfg["vocab_size"], 7000 + i) for i, n in zip(ids, lens)]
    expect = [oracle.logits(q) for q in seqs]
    for slots, shape in ((19 + 7, 24), (19, 19)):
        runner = ModelRunner(model, page_size=8, num_pages=160, num_slots=slots, pad_decode=True)
        for r, n, q in zip(ids, lens, seqs):
            runner.admit(r)
            runner.step([StepEntry(r, q[:n], [])])
        live = list(ids)
        for j in range(new):
            if j == 3:                               # two requests end: 17 are left
                for r in (4, 11):
                    runner.release(r)
                    live.remove(r)
            logits = runner.step([StepEntry(r, [seqs[r][lens[r] + j]], [0]) for r in live])
            assert logits.shape[0] == len(live)
            for row, r in enumerate(live):
                err = eu.rel_err(logits[row], expect[r][lens[r] + j])
                assert err < TOL[dtype], f"{slots} slots, step {j}, request {r}: off by {err:.3e}"
        sizes = {key[0] for key in runner.graphs.entries}
        assert sizes == ({shape} if shape == 24 else {19, 17}), sizes
        if shape == 24:
            assert runner.graphs.captures == 1 and runner.graphs.replays == new - 1
        for r in live:
            runner.release(r)
        runner.release_padding()
        runner.cache.check()
        stats = runner.cache.stats()
        assert stats["requests"] == 0 and stats["slots_free"] == stats["slots"]
        assert all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_a_batch_that_stays_gets_a_recording_of_its_own(monkeypatch):
    """A batch that is filled up with padding rows runs them at every step; once it has come
    as it is more often than ``PROMOTE_AFTER`` it is recorded without them."""
    from zig_ai_amd.engine import ModelRunner, StepEntry, graphs
    monkeypatch.setattr(graphs, "PROMOTE_AFTER", 2)
    model, _, _ = setup("D", "float32")
    cfg, seed = CONFIGS["D"]
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, torch.float32, **eu.sharp_kwargs()))
    ids = list(range(19))
    new = 7
    seqs = [eu.random_tokens(4 + r % 5 + new, cfg["vocab_size"], 7300 + r) for r in ids]
    expect = [oracle.logits(q) for q in seqs]
    runner = ModelRunner(model, page_size=8, num_pages=160, num_slots=19 + 7, pad_decode=True)
    for r, q in zip(ids, seqs):
        runner.admit(r)
        runner.step([StepEntry(r, q[:len(q) - new], [])])
    sizes = []
    for j in range(new):
        logits = runner.step([StepEntry(r, [seqs[r][len(seqs[r]) - new + j]], [0]) for r in ids])
        for r in ids:
            assert eu.rel_err(logits[r], expect[r][len(seqs[r]) - new + j]) < TOL["float32"], (j, r)
        sizes.append(sorted(key[0] for key, slot in runner.graphs.entries.items()
                            if slot["graph"] is not None))
    # two steps filled up to 24 (the second records that shape), then the batch of 19 as it
    # is: run, recorded, replayed
    assert sizes == [[], [24], [24], [19, 24], [19, 24], [19, 24], [19, 24]], sizes
    assert runner.graphs.captures == 2 and runner.graphs.replays == 1 + 4


def test_padding_rows_give_their_pages_back_when_requests_need_them():
    """17 requests and 7 padding rows in a pool with ten pages to spare: when every request
    needs its second page the padding rows' pages are what is missing; they are given back,
    the step runs without them, and so do the later ones (no page is left for such rows)."""
    from zig_ai_amd.engine import ModelRunner, StepEntry
    model, _, _ = setup("A", "float32")
    cfg, seed = CONFIGS["A"]
    oracle = plain.PlainLfm2(eu.model_folder(cfg, seed, torch.float32, **eu.sharp_kwargs()))
    ids = list(range(17))
    seqs = [eu.random_tokens(3 + 4, cfg["vocab_size"], 7100 + i) for i in ids]
    expect = [oracle.logits(q) for q in seqs]
    runner = ModelRunner(model, page_size=4, num_pages=17 + 7 + 10, num_slots=24, pad_decode=True)
    runner.PAD_SPARE_PAGES = 0               # (by itself a runner takes no such rows in so small a pool)
    for r, q in zip(ids, seqs):
        runner.admit(r)
        runner.step([StepEntry(r, q[:3], [])])
    shapes = []
    for j in range(4):
        logits = runner.step([StepEntry(r, [seqs[r][3 + j]], [0]) for r in ids])
        shapes.append(len(runner._pads))
        for r in ids:
            assert eu.rel_err(logits[r], expect[r][3 + j]) < TOL["float32"], (j, r)
        runner.cache.check()
    # position 3 fills the first page (7 rows beside the requests), position 4 needs the second
    assert shapes == [7, 0, 0, 0]
    assert {key[0] for key in runner.graphs.entries} == {24, 17}
    for r in ids:
        runner.release(r)
    runner.release_padding()
    stats = runner.cache.stats()
    assert stats["requests"] == 0 and all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_recorded_shapes_are_dropped_when_there_are_too_many(monkeypatch):
    """Only so many recorded steps are kept; the one used longest ago goes, and comes
    back (recorded anew) when its shape does.  Three batch sizes in turn, three steps
    each, with room for two: every step still gives the plain implementation's logits."""
    from zig_ai_amd.engine import StepEntry, graphs
    monkeypatch.setattr(graphs, "MAX_GRAPHS", 2)
    model, expect, prompts = setup("B", "float32")
    runner = runner_for(model, 8, 64, num_slots=4)
    live = [4, 3, 2]                                   # 100, 64 and 31 tokens
    got = {i: [] for i in live}
    cursor = {}
    for i in live:
        runner.admit(i)
        got[i].append(runner.step([StepEntry(i, prompts[i][:20], list(range(20)))]).cpu())
        cursor[i] = 20
    for step in range(33):
        # batch sizes 1, 1, 1, 2, 2, 2, 3, 3, 3, 1 ...: a shape's first step runs
        # unrecorded, its second is recorded and replayed, its third replayed
        members = live[:1 + (step // 3) % 3]
        members = [i for i in members if cursor[i] < len(prompts[i])]
        if not members:
            break
        out = runner.step([StepEntry(i, [prompts[i][cursor[i]]], [0]) for i in members]).cpu()
        for row, i in enumerate(members):
            got[i].append(out[row:row + 1])
            cursor[i] += 1
        assert len(runner.graphs.entries) <= 2
    assert runner.graphs.captures > 3                  # shapes were recorded again
    assert runner.graphs.replays >= 2 * runner.graphs.captures - 1
    for i in live:
        have = torch.cat(got[i])
        assert eu.rel_err(have, expect[i][:have.shape[0]]) < TOL["float32"]


def random_case(seed: int):
    """A random small LFM2 configuration, requests, page size and way of cutting."""
    import random
    rng = random.Random(seed)
    d = rng.choice([16, 32, 48, 64, 64, 128])
    nkv = rng.choice([1, 2, 3])
    nh = nkv * rng.choice([1, 2, 4, 5] if d <= 64 else [1, 2])
    layers = rng.randint(2, 5)
    types = [rng.choice(["conv", "full_attention"]) for _ in range(layers)]
    if "full_attention" not in types:
        types[rng.randrange(layers)] = "full_attention"
    if "conv" not in types:
        types[rng.randrange(layers)] = "conv"
    cfg = {"architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
           "hidden_size": rng.choice([64, 96, 128, 160, 200]), "num_hidden_layers": layers,
           "num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d,
           "vocab_size": rng.randint(40, 700), "layer_types": types,
           "intermediate_size": 8 * rng.randint(5, 40), "rope_theta": rng.choice([1e4, 1e6]),
           "norm_eps": rng.choice([1e-5, 1e-6]), "conv_L_cache": rng.randint(1, 6),
           "conv_bias": rng.random() < 0.5, "tie_embedding": rng.random() < 0.5,
           "max_position_embeddings": 4096}
    lengths = [rng.choice([1, 2, 3, 9, 17, 40, 77, 130, 200]) for _ in range(rng.randint(2, 5))]
    page = rng.choice([4, 8, 16, 32])
    kind = rng.choice(["whole", "bulk", "portions", "mixed"])
    if kind == "whole":
        schedule = eu.whole(lengths)
    elif kind == "bulk":
        schedule = eu.bulk_then_single(lengths, rng.choice([5, 32]))
    elif kind == "portions":
        schedule = eu.changing_portions(lengths, rng.randrange(9))
    else:
        schedule = eu.mixed(lengths, seed=rng.randrange(100), max_live=rng.choice([2, 3, 4]))
    pages = eu.peak_tokens(lengths, schedule, round_to=page) // page
    return cfg, lengths, page, pages, schedule


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations_and_cuts(seed):
    """Sixteen configurations drawn at random (head sizes 16 to 128, one to fifteen
    query heads in groups of one to five, convolution lengths 1 to 6, with and without
    biases and tied heads, vocabularies and widths that are no powers of two), each with
    its own requests, page size and way of cutting the work: in 32-bit the engine is the
    plain implementation to 1e-4, whatever the draw; bfloat16 stays within its tolerance."""
    from zig_ai_amd.engine import DecoderModel, ModelRunner
    cfg, lengths, page, pages, schedule = random_case(seed)
    for dtype in ("float32", "bfloat16"):
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = eu.model_folder(cfg, seed, store, **eu.sharp_kwargs())
        model = DecoderModel.from_folder(folder, dtype)
        oracle = plain.PlainLfm2(folder)
        prompts = [eu.random_tokens(n, cfg["vocab_size"], 31 * seed + i) for i, n in enumerate(lengths)]
        expect = [oracle.logits(p) for p in prompts]
        runner = ModelRunner(model, page_size=page, num_pages=pages, num_slots=4)
        model.layer_oracle = oracle if dtype == "float32" else plain.PlainLfm2(folder, dtype=torch.float32)
        run_and_check(model, runner, prompts, expect, schedule, dtype, f"seed {seed}")
        assert runner.cache.stats()["requests"] == 0
