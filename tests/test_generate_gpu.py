"""Generation through the entry points (Python API, command line, trace replay)
against the plain implementation, and the scheduler's behaviour on the GPU when
pages run out."""

import json
import os
import subprocess
import sys

import pytest
import torch

import engine_util as eu
import plain_lfm2 as plain
from tiny_configs import TINY_A, TINY_B, TINY_D

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def folder_for(cfg, seed, dtype=torch.float32, weights="sharp"):
    """``sharp``: the weights under which faults show (see ``engine_util.sharp_kwargs``).
    ``as written``: what the workloads' definitions say, every matrix N(0, 0.02), with norm
    weights of 1 (tiny-A) or drawn like everything else (``all normal``, tiny-B)."""
    if weights == "sharp":
        return eu.model_folder(cfg, seed, dtype, **eu.sharp_kwargs())
    return eu.model_folder(cfg, seed, dtype, std=0.02,
                           norm_init="ones" if weights == "as written" else "normal")


@pytest.mark.parametrize("weights", ["sharp", "as written"])
def test_greedy_generation_tiny_a(weights):
    """The tiny-A workload: prompts of 5/17/33 tokens, 16 greedy tokens each,
    page size 4, in 32-bit, seed 0: the same tokens as the plain implementation."""
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_A, 0, weights=weights)
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 256, 200 + n) for n in (5, 17, 33)]
    engine = Engine(folder, dtype="float32", page_size=4, num_pages=64, max_num_seqs=4)
    got = engine.generate(prompts, max_new_tokens=16, temperature=0.0, eos_token_id=-1)
    for p, g in zip(prompts, got):
        assert g == oracle.greedy(p, 16)
    stats = engine.stats()
    assert stats["requests"] == 0 and stats["slots_free"] == stats["slots"]
    assert all(g["pages_free"] == g["pages"] for g in stats["groups"])


def follow_sampling(oracle, prompt, tokens, params, number):
    """Check a sampled continuation token by token against the plain sampler fed
    with the same uniform numbers."""
    from zig_ai_amd.sampling import UniformStream
    stream = UniformStream(params["seed"], number)
    seq = list(prompt)
    for k, tok in enumerate(tokens):
        logits = oracle.logits(seq)[-1]
        history = seq[len(prompt):]
        if params.get("repetition_penalty", 1.0) != 1.0:
            logits = plain.apply_repetition_penalty(logits, history, params["repetition_penalty"])
        want = plain.sample_token(logits, params["temperature"], stream.at(k),
                                  params.get("top_k", 0), params.get("top_p", 1.0))
        assert tok == want, f"token {k}: engine {tok}, plain {want}"
        seq.append(tok)


@pytest.mark.parametrize("params", [
    dict(temperature=0.7, seed=1234),
    dict(temperature=0.7, seed=1234, weights="as written"),
    dict(temperature=0.7, seed=1234, weights="all normal"),
    dict(temperature=1.3, top_k=20, seed=7),
    dict(temperature=0.9, top_p=0.8, seed=8),
    dict(temperature=0.8, top_k=50, top_p=0.9, repetition_penalty=1.3, seed=9),
    dict(temperature=0.0, repetition_penalty=1.5, seed=1),
])
def test_sampled_generation_tiny_b(params):
    """The tiny-B workload: prompts of 1/8/31/64/100 tokens, chunked prefill of
    16, temperature 0.7 with a fixed sampling seed, page size 8; and the sampler's
    other options."""
    from zig_ai_amd.engine import Engine
    params = dict(params)
    folder = folder_for(TINY_B, 1, weights=params.pop("weights", "sharp"))
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 512, 300 + n) for n in (1, 8, 31, 64, 100)]
    engine = Engine(folder, dtype="float32", page_size=8, num_pages=128, max_num_seqs=8,
                    chunk_size=16, max_num_batched_tokens=40)
    got = engine.generate(prompts, max_new_tokens=10, eos_token_id=-1, **params)
    for number, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == 10
        follow_sampling(oracle, p, g, params, number)


# A bfloat16 run's logits lie within about one percent of the plain implementation's
# (of the largest logit); what is drawn from them is held to that.
BF16_NEAR = 1e-2


def follow_bfloat16(oracle, prompt, tokens, params, number):
    """A continuation generated in bfloat16, token by token along the ENGINE's tokens, against
    the plain implementation's 64-bit logits for the same history.  Greedy: the chosen token's
    plain logit is within ``BF16_NEAR`` (of the largest logit) of the plain maximum.  Sampled:
    with the request's own uniform number ``u`` for that token, ``u`` lies in the chosen
    token's interval of the plain cumulative distribution, widened by what logits off by
    ``BF16_NEAR`` can move the distribution's edges.  Returns the largest distance seen."""
    from zig_ai_amd.sampling import UniformStream
    stream = UniformStream(params.get("seed", 42), number)
    seq = list(prompt)
    worst = 0.0
    T = params["temperature"]
    for k, tok in enumerate(tokens):
        logits = oracle.logits(seq)[-1].double()
        scale = float(logits.abs().max())
        if T <= 0:
            gap = float(logits.max() - logits[tok]) / scale
            assert gap <= BF16_NEAR, f"token {k}: engine chose {tok}, {gap:.2e} below the plain maximum"
            worst = max(worst, gap)
        else:
            p = torch.softmax(logits / T, dim=0)
            hi = float(p[:tok + 1].sum())
            lo = hi - float(p[tok])
            # every logit off by at most e: every probability by a factor within exp(+-2e/T)
            slack = float(torch.expm1(torch.tensor(2.0 * BF16_NEAR * scale / T)))
            u = stream.at(k)
            assert lo - slack <= u <= hi + slack, \
                f"token {k}: u = {u:.4f} outside [{lo:.4f}, {hi:.4f}] +- {slack:.3f} of token {tok}"
            worst = max(worst, lo - u, u - hi, 0.0)
        seq.append(tok)
    return worst


@pytest.mark.parametrize("temperature", [0.0, 0.7])
@pytest.mark.parametrize("name", ["B", "D"])
def test_generation_in_bfloat16_through_scheduler_and_graphs(name, temperature):
    """bfloat16 through everything serving uses at once: the scheduler (prompts in portions,
    requests that join late), up to eight decode steps issued ahead with the tokens handed
    over on the device, recorded graphs, the sampler on the device.  Each generated token
    is checked against the plain implementation given the same history."""
    from zig_ai_amd.engine import Engine
    cfg, seed, lens = {"B": (TINY_B, 1, (1, 8, 31, 64, 100)), "D": (TINY_D, 3, (150, 9, 66, 40))}[name]
    # tiny-B's weights as its workload writes them; D (matrix-core attention) with the
    # weights under which a misplaced key would show
    folder = folder_for(cfg, seed, torch.bfloat16, weights="as written" if name == "B" else "sharp")
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, cfg["vocab_size"], 500 + n) for n in lens]
    engine = Engine(folder, dtype="bfloat16", page_size=8, num_pages=128, max_num_seqs=3,
                    chunk_size=16, max_num_batched_tokens=40, multi_step=8)
    params = dict(temperature=temperature, seed=1234)
    got = engine.generate(prompts, max_new_tokens=24, eos_token_id=-1, **params)
    for number, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == 24
        follow_bfloat16(oracle, p, g, params, number)
    graphs = engine.runner.graphs
    assert graphs is not None and graphs.replays >= 24, "the decode steps were not replayed"
    stats = engine.stats()
    assert stats["requests"] == 0 and all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_an_engine_takes_a_model_that_is_already_built():
    """``Engine`` around ``DecoderModel.from_random``: no folder on the way."""
    from zig_ai_amd.engine import DecoderModel, Engine
    model = DecoderModel.from_random(TINY_A, seed=0, dtype="float32", **eu.sharp_kwargs())
    folder = folder_for(TINY_A, 0)
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 256, 200 + n) for n in (5, 17)]
    engine = Engine(model, page_size=4, num_pages=64, max_num_seqs=4)
    got = engine.generate(prompts, max_new_tokens=8, temperature=0.0, eos_token_id=-1)
    assert got == [oracle.greedy(p, 8) for p in prompts]


def test_tokens_do_not_depend_on_scheduling():
    """Other budgets, portion sizes, page sizes, and a pool so small that requests
    are preempted and recomputed: the same tokens."""
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_B, 1)
    prompts = [eu.random_tokens(n, 512, 400 + n) for n in (30, 12, 45, 7, 60, 22)]
    kw = dict(max_new_tokens=24, temperature=0.8, top_k=40, seed=5, eos_token_id=-1)
    base = Engine(folder, dtype="float32", page_size=16, num_pages=64).generate(prompts, **kw)
    other = Engine(folder, dtype="float32", page_size=4, num_pages=200, chunk_size=5,
                   max_num_batched_tokens=11, max_num_seqs=3).generate(prompts, **kw)
    assert other == base
    tight = Engine(folder, dtype="float32", page_size=4, num_pages=30, chunk_size=16,
                   max_num_batched_tokens=64, max_num_seqs=6)
    assert tight.generate(prompts, **kw) == base
    stats = tight.stats()
    assert stats["preemptions"] > 0, "the pool was large enough that nothing was preempted"
    assert stats["requests"] == 0
    assert all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_decode_batches_filled_up_to_recorded_sizes():
    """28 requests that stop one after the other: above 16 requests the decode batch is
    filled up to a multiple of 8 with rows of the engine's own, so the batches of 28 down
    to 17 requests meet two recorded shapes instead of twelve.  The tokens are those of an
    engine that records nothing; the rows' slots and pages are back when no request is left."""
    from zig_ai_amd.engine import Engine
    from zig_ai_amd.sampling.sampler import SamplingParams
    folder = folder_for(TINY_B, 1)
    prompts = [eu.random_tokens(3 + (5 * i) % 17, 512, 900 + i) for i in range(28)]
    lengths = [6 + i for i in range(28)]
    for sampling in (SamplingParams(temperature=0.0), SamplingParams(temperature=0.9, top_k=50, seed=8)):
        def run(engine):
            reqs = [engine.add_request(p, n, sampling, eos_token_id=-1) for p, n in zip(prompts, lengths)]
            engine.run()
            return [list(r.output) for r in reqs]
        kw = dict(dtype="float32", page_size=8, num_pages=256, max_num_seqs=28)
        want = run(Engine(folder, use_graphs=False, **kw))
        engine = Engine(folder, **kw)
        assert run(engine) == want
        graphs = engine.runner.graphs
        sizes = sorted({key[0] for key in graphs.entries})
        assert [n for n in sizes if n > 16] == [24, 32], sizes
        assert graphs.replays >= 12          # of the 16 steps with more than 16 requests
        stats = engine.stats()
        assert stats["requests"] == 0 and stats["slots_free"] == stats["slots"]
        assert all(g["pages_free"] == g["pages"] for g in stats["groups"])
        engine.runner.cache.check()


def test_the_engine_warms_up_before_its_first_request():
    """A bfloat16 engine whose projections are large enough to be timed runs one step of
    every block of row counts up to its token budget when it is made, with a request of
    its own that leaves nothing behind; a 32-bit engine, and one whose model takes the
    library's first answer, have nothing to warm up."""
    from zig_ai_amd.engine import DecoderModel, Engine
    from tiny_configs import REAL_350M_2L
    model = DecoderModel.from_random(REAL_350M_2L, seed=0, dtype="bfloat16", quick=True)
    engine = Engine(model, page_size=16, num_pages=512, max_num_seqs=8, max_num_batched_tokens=600)
    # 24 ... 64 (the sizes decode batches are filled up to), 128, 255, 256, 512
    assert engine.warm_up_steps == 10
    stats = engine.stats()
    assert stats["requests"] == 0 and stats["slots_free"] == stats["slots"]
    assert all(g["pages_free"] == g["pages"] for g in stats["groups"])
    out = engine.generate([eu.random_tokens(40, REAL_350M_2L["vocab_size"], 3)], max_new_tokens=4,
                          temperature=0.0, eos_token_id=-1)
    assert len(out[0]) == 4
    fixed = DecoderModel.from_random(REAL_350M_2L, seed=0, dtype="bfloat16", quick=True, reproducible=True)
    assert Engine(fixed, page_size=16, num_pages=512, max_num_seqs=8).warm_up_steps == 0
    assert Engine(folder_for(TINY_A, 0), dtype="float32", page_size=4, num_pages=64).warm_up_steps == 0


def test_a_length_limit_beyond_the_models_own_is_refused():
    """``max_model_len`` above the model's ``max_position_embeddings`` would stop a step in
    the middle of a call and every request of the call with it: refused when the engine is
    made."""
    from zig_ai_amd.engine import Engine
    short = dict(TINY_A, max_position_embeddings=64)
    folder = eu.model_folder(short, 0, torch.float32, **eu.sharp_kwargs())
    with pytest.raises(ValueError, match="max_position_embeddings"):
        Engine(folder, dtype="float32", page_size=4, num_pages=64, max_model_len=100)
    engine = Engine(folder, dtype="float32", page_size=4, num_pages=64)
    assert engine.max_model_len == 64
    with pytest.raises(ValueError):
        engine.generate([eu.random_tokens(60, 256, 1)], max_new_tokens=10, temperature=0.0)
    assert len(engine.generate([eu.random_tokens(50, 256, 1)], max_new_tokens=10,
                               temperature=0.0, eos_token_id=-1)[0]) == 10


def test_eos_and_length_stop():
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_A, 0)
    engine = Engine(folder, dtype="float32", page_size=4, num_pages=64, max_num_seqs=4)
    prompt = eu.random_tokens(9, 256, 1)
    free_run = engine.generate([prompt], max_new_tokens=12, temperature=0.0, eos_token_id=-1)[0]
    stop_at = free_run[4]
    first = free_run.index(stop_at)
    stopped = engine.generate([prompt], max_new_tokens=12, temperature=0.0, eos_token_id=stop_at)[0]
    assert stopped == free_run[:first + 1]
    assert engine.generate([prompt], max_new_tokens=0, temperature=0.0)[0] == []


def test_steps_issued_ahead_change_nothing():
    """Up to 8 decode steps issued without waiting for the tokens in between, against
    one step at a time: the same tokens, also for a request that meets its stop token
    in the middle of such a run, with sampling and with a budget that admits late."""
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_B, 1)
    prompts = [eu.random_tokens(n, 512, 600 + n) for n in (12, 40, 7, 25)]
    for kw in (dict(temperature=0.0), dict(temperature=0.9, top_k=30, seed=11)):
        def one():                                    # a new engine: requests numbered from 0
            return Engine(folder, dtype="float32", page_size=8, num_pages=64, max_num_seqs=4,
                          multi_step=1)
        free_run = one().generate(prompts, max_new_tokens=20, eos_token_id=-1, **kw)
        stop = free_run[1][9]                         # request 1 stops inside a run of 8
        want = one().generate(prompts, max_new_tokens=20, eos_token_id=stop, **kw)
        ahead = Engine(folder, dtype="float32", page_size=8, num_pages=64, max_num_seqs=2,
                       multi_step=8)                  # two at a time: the others wait, then join
        got = ahead.generate(prompts, max_new_tokens=20, eos_token_id=stop, **kw)
        assert got == want and len(want[1]) <= 10
        stats = ahead.stats()
        assert stats["requests"] == 0 and all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_runs_of_steps_issued_before_the_last_run_is_read():
    """Runs of 3 decode steps, the next run issued before the tokens of the last one are
    read: a request that meets its stop token in one run while the next is already on the
    GPU, requests that reach their lengths at different steps, and so few pages that a
    run ends early and a request is preempted; always the tokens of one step at a time."""
    from zig_ai_amd.engine import Engine
    from zig_ai_amd.sampling.sampler import SamplingParams
    folder = folder_for(TINY_B, 1)
    prompts = [eu.random_tokens(n, 512, 640 + n) for n in (12, 30, 7)]
    for kw in (dict(temperature=0.0), dict(temperature=0.8, top_p=0.95, seed=5)):
        def engine(multi_step, num_pages=64):         # a new engine: requests numbered from 0
            return Engine(folder, dtype="float32", page_size=8, num_pages=num_pages, max_num_seqs=3,
                          multi_step=multi_step)
        free_run = engine(1).generate(prompts, max_new_tokens=30, eos_token_id=-1, **kw)
        stop = free_run[2][7]                         # request 2 stops in the third run of 3
        want = engine(1).generate(prompts, max_new_tokens=30, eos_token_id=stop, **kw)
        assert len(want[2]) <= 8
        ahead = engine(3)
        assert ahead.generate(prompts, max_new_tokens=30, eos_token_id=stop, **kw) == want
        assert ahead.runner.graphs.replays > 20
        stats = ahead.stats()
        assert stats["requests"] == 0 and all(g["pages_free"] == g["pages"] for g in stats["groups"])
        # requests with different lengths left: the run is as long as the shortest allows
        sampling = SamplingParams(temperature=kw["temperature"], top_p=kw.get("top_p", 1.0),
                                  seed=kw.get("seed", 42))

        def uneven(e):
            reqs = [e.add_request(p, n, sampling, eos_token_id=-1) for p, n in zip(prompts, (30, 11, 23))]
            e.run()
            return [list(r.output) for r in reqs]
        got = uneven(engine(3))
        assert got == uneven(engine(1)) and [len(g) for g in got] == [30, 11, 23]
        # a call of step() returns after a bounded number of runs: a request added between
        # two calls joins then
        calls = engine(2)
        calls.RUNS_PER_CALL = 2
        first = calls.add_request(prompts[0], 30, sampling, eos_token_id=-1)
        calls.step()                                  # the prompt
        before = calls.stats()["steps"]
        calls.step()
        assert calls.stats()["steps"] - before == 4
        second = calls.add_request(prompts[1], 11, sampling, eos_token_id=-1)
        calls.run()
        assert [first.output, second.output] == got[:2]
        # 14 pages of 8 tokens: the three requests need 6 + 6 + 4 at their ends
        tight = engine(3, num_pages=14)
        assert tight.generate(prompts, max_new_tokens=30, eos_token_id=-1, **kw) == free_run
        assert tight.stats()["preemptions"] >= 1
        stats = tight.stats()
        assert stats["requests"] == 0 and all(g["pages_free"] == g["pages"] for g in stats["groups"])


def test_command_line_greedy():
    folder = folder_for(TINY_A, 0)
    oracle = plain.PlainLfm2(folder)
    prompt = eu.random_tokens(11, 256, 77)
    out = subprocess.run(
        [sys.executable, "-m", "zig_ai_amd", "-m", folder, "--prompt", " ".join(map(str, prompt)),
         "-n", "8", "--temperature", "0", "--dtype", "float32", "--page-size", "4",
         "--num-pages", "32", "--max-num-seqs", "2", "--eos", "-1", "--json"],
        cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    result = json.loads(out.stdout.strip().splitlines()[-1])
    assert result["outputs"] == [oracle.greedy(prompt, 8)]


def test_command_line_diagnostics(tmp_path):
    """--random-weights with --config, --no-graph, --dump-logits, --verbose, --profile:
    the same tokens with and without graphs; the dumped logits are those of the plain
    implementation on the random model the same seed writes."""
    import numpy as np
    from tiny_configs import TINY_B
    from zig_ai_amd.config import config_from_dict
    from zig_ai_amd.weights import write_random_model
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY_B))
    prompt = eu.random_tokens(9, 512, 78)
    base = [sys.executable, "-m", "zig_ai_amd", "--random-weights", "--config", str(cfg_path),
            "--weights-seed", "5", "--prompt-ids", " ".join(map(str, prompt)), "-n", "6",
            "--temperature", "0", "--dtype", "float32", "--page-size", "8", "--num-pages", "16",
            "--max-num-seqs", "2", "--eos", "-1", "--json"]
    dump = tmp_path / "dump"
    runs = []
    for extra in (["--no-graph", "--dump-logits", str(dump), "--verbose", "--profile"], []):
        out = subprocess.run(base + extra, cwd=ROOT, capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-2000:]
        runs.append((json.loads(out.stdout.strip().splitlines()[-1])["outputs"], out.stderr))
    assert runs[0][0] == runs[1][0]
    assert "step 0: 1 requests, 9 tokens" in runs[0][1] and "decode:" in runs[0][1]
    folder = str(tmp_path / "model")
    write_random_model(config_from_dict(TINY_B), folder, seed=5, dtype=torch.float32)
    oracle = plain.PlainLfm2(folder)
    assert runs[0][0] == [oracle.greedy(prompt, 6)]
    seq = list(prompt)
    for step in range(6):
        got = torch.from_numpy(np.fromfile(dump / f"{step}.f32", dtype="<f4"))
        assert eu.rel_err(got.view(1, -1), oracle.logits(seq)[-1:]) < 1e-4
        seq.append(runs[0][0][0][step])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["whole", "bulk", "portions", "mixed"])
def test_trace_run(dtype, kind, tmp_path):
    """bin/trace_run on the same requests whole, with the last 32 tokens one by one, in
    portions of changing size, and mixed with a pool so small that pages are used again;
    every wanted row, found through index.json, against the plain implementation."""
    import numpy as np
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = folder_for(TINY_B, 1, store)
    oracle = plain.PlainLfm2(folder)
    lengths = [70, 33, 100, 18, 64, 90]
    prompts = [eu.random_tokens(n, 512, 500 + i) for i, n in enumerate(lengths)]
    schedule = {"whole": eu.whole(lengths), "bulk": eu.bulk_then_single(lengths, 32),
                "portions": eu.changing_portions(lengths, 2),
                "mixed": eu.mixed(lengths, seed=4, max_live=4)}[kind]
    lines, wanted = [], {}
    for step, (entries, ends) in enumerate(schedule):
        rec = {"step": step, "entries": [], "end": [f"r{i}" for i in ends]}
        for i, a, b in entries:
            want = [k for k in range(b - a) if (a + k) % 3 != 1]        # not every place
            rec["entries"].append({"id": f"r{i}", "tokens": prompts[i][a:b], "want": want})
            wanted.setdefault(f"r{i}", []).extend(a + k for k in want)
        lines.append(json.dumps(rec))
    out_dir = tmp_path / "out"
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(eu.peak_tokens(lengths, schedule, 64))],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == [w for s in range(len(schedule)) for w in ("done", str(s))]
    with open(out_dir / "index.json") as f:
        index = json.load(f)
    assert {r: [p for p, _, _ in rows] for r, rows in index.items()} == wanted
    tol = 1e-4 if dtype == "float32" else 4e-2
    files = {}
    for i, p in enumerate(prompts):
        expect = oracle.logits(p)
        got = []
        for place, step, row in index[f"r{i}"]:
            if step not in files:
                files[step] = torch.from_numpy(np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(-1, 512))
            got.append(files[step][row])
        err = eu.rel_err(torch.stack(got), expect[[place for place, _, _ in index[f"r{i}"]]])
        assert err < tol, f"request {i}: {err:.3e}"
    for step, (entries, _) in enumerate(schedule):       # a step that wants nothing writes nothing
        rows = sum(1 for i, a, b in entries for k in range(a, b) if k % 3 != 1)
        assert (out_dir / f"{step}.f32").exists() == (rows > 0)
        if rows:
            assert files[step].shape[0] == rows


def test_trace_run_with_random_weights(tmp_path):
    """``--config FILE --random-weights --seed S`` replays on the model that the random model
    writer stores for that configuration and seed."""
    import numpy as np
    from zig_ai_amd.weights import write_random_model
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(TINY_A))
    folder = str(tmp_path / "model")
    write_random_model(TINY_A, folder, seed=9, dtype=torch.float32)
    prompt = eu.random_tokens(21, 256, 77)
    trace = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": prompt[:13], "want": [12]}], "end": []}) \
        + "\n" + json.dumps({"step": 1, "entries": [{"id": "a", "tokens": prompt[13:], "want": [0, 7]}],
                             "end": ["a"]}) + "\n"
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--config", str(cfg_path), "--random-weights",
         "--seed", "9", "--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "64"],
        input=trace, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    expect = plain.PlainLfm2(folder).logits(prompt)
    got = torch.cat([torch.from_numpy(np.fromfile(tmp_path / "out" / f"{s}.f32", dtype="<f4").reshape(-1, 256))
                     for s in (0, 1)])
    assert eu.rel_err(got, expect[[12, 13, 20]]) < 1e-4
    assert json.load(open(tmp_path / "out" / "index.json")) == {"a": [[12, 0, 0], [13, 1, 0], [20, 1, 1]]}
    bad = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--dtype", "float32", "--out",
                          str(tmp_path / "o2"), "--max-tokens", "64"], input="", capture_output=True, text=True)
    assert bad.returncode != 0 and "--model" in bad.stderr


def test_an_engine_used_again_and_again_keeps_nothing():
    """Forty calls of generate() on one engine, with other batch sizes, lengths and
    sampling options each time and a pool that forces preemptions now and then:
    afterwards no request, page, slot or name is held, and device memory has not
    grown since the first calls."""
    import random

    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_B, 1)
    engine = Engine(folder, dtype="bfloat16", page_size=8, num_pages=48, max_num_seqs=5,
                    chunk_size=32, max_num_batched_tokens=80)
    rng = random.Random(3)
    allocated = []
    for call in range(40):
        n = rng.randint(1, 7)
        prompts = [eu.random_tokens(rng.randint(1, 90), 512, 1000 * call + i) for i in range(n)]
        kw = rng.choice([dict(temperature=0.0), dict(temperature=0.8, seed=call),
                         dict(temperature=1.1, top_k=20, top_p=0.9, seed=call),
                         dict(temperature=0.0, repetition_penalty=1.2)])
        new = rng.randint(1, 24)
        out = engine.generate(prompts, max_new_tokens=new, eos_token_id=-1, **kw)
        assert [len(o) for o in out] == [new] * n
        stats = engine.stats()
        assert stats["requests"] == 0
        assert all(g["pages_free"] == g["pages"] for g in stats["groups"])
        assert stats["slots_free"] == stats["slots"]
        assert len(engine.runner.cache.handles) == 0
        torch.cuda.synchronize()
        allocated.append(torch.cuda.memory_allocated())
    assert engine.stats()["preemptions"] > 0
    assert max(allocated[20:]) <= max(allocated[:20])


def test_a_failed_generate_leaves_nothing_behind():
    """One request of the call can never fit the pool: generate() raises, and what the
    other requests of that call held is given back; the engine then serves the next call
    as if nothing had happened."""
    from zig_ai_amd.cache import OutOfPages
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_B, 1)
    oracle = plain.PlainLfm2(folder)
    engine = Engine(folder, dtype="float32", page_size=8, num_pages=6, max_num_seqs=4,
                    max_model_len=400)
    small = [eu.random_tokens(n, 512, 70 + n) for n in (5, 9)]
    too_long = eu.random_tokens(60, 512, 99)             # 60 tokens need 8 pages; there are 6
    with pytest.raises(OutOfPages):
        engine.generate(small + [too_long], max_new_tokens=4, temperature=0.0, eos_token_id=-1)
    stats = engine.stats()
    assert stats["requests"] == 0 and stats["slots_free"] == stats["slots"]
    assert all(g["pages_free"] == g["pages"] for g in stats["groups"])
    assert len(engine.runner.cache.handles) == 0
    got = engine.generate(small, max_new_tokens=5, temperature=0.0, eos_token_id=-1)
    assert got == [oracle.greedy(p, 5) for p in small]
    with pytest.raises(ValueError):                      # refused on entry: also nothing left
        engine.generate(small + [[1] * 500], max_new_tokens=4, temperature=0.0)
    assert engine.stats()["requests"] == 0 and len(engine.runner.cache.handles) == 0


def test_command_line_says_what_is_wrong(tmp_path):
    """No such folder, a folder without weights, a token outside the vocabulary: one
    line on standard error and exit status 1, no traceback."""
    folder = folder_for(TINY_A, 0)
    empty = tmp_path / "empty"
    empty.mkdir()
    (empty / "config.json").write_text(open(os.path.join(folder, "config.json")).read())
    cases = [(["-m", str(tmp_path / "nowhere"), "--prompt-ids", "1 2"], "nowhere"),
             (["-m", str(empty), "--prompt-ids", "1 2"], "safetensors"),
             (["-m", folder, "--prompt-ids", "1 999999", "--dtype", "float32"], "999999")]
    for args, word in cases:
        out = subprocess.run([sys.executable, "-m", "zig_ai_amd"] + args + ["-n", "2"], cwd=ROOT,
                             capture_output=True, text=True, timeout=600)
        assert out.returncode == 1, (args, out.stderr[-500:])
        assert "Traceback" not in out.stderr and word in out.stderr, (args, out.stderr[-500:])
        assert out.stderr.strip().splitlines()[-1].startswith("zig-ai: ")
