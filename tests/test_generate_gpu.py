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
from tiny_configs import TINY_A, TINY_B

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def folder_for(cfg, seed, dtype=torch.float32):
    return eu.model_folder(cfg, seed, dtype, **eu.sharp_kwargs())


def test_greedy_generation_tiny_a():
    """The tiny-A workload: prompts of 5/17/33 tokens, 16 greedy tokens each,
    page size 4, in 32-bit: the same tokens as the plain implementation."""
    from zig_ai_amd.engine import Engine
    folder = folder_for(TINY_A, 0)
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
    folder = folder_for(TINY_B, 1)
    oracle = plain.PlainLfm2(folder)
    prompts = [eu.random_tokens(n, 512, 300 + n) for n in (1, 8, 31, 64, 100)]
    engine = Engine(folder, dtype="float32", page_size=8, num_pages=128, max_num_seqs=8,
                    chunk_size=16, max_num_batched_tokens=40)
    got = engine.generate(prompts, max_new_tokens=10, eos_token_id=-1, **params)
    for number, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == 10
        follow_sampling(oracle, p, g, params, number)


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
def test_trace_run(dtype, tmp_path):
    """bin/trace_run on a mixed trace with a pool so small that pages are used
    again; every wanted row against the plain implementation."""
    import numpy as np
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = folder_for(TINY_B, 1, store)
    oracle = plain.PlainLfm2(folder)
    lengths = [70, 33, 100, 18, 64, 90]
    prompts = [eu.random_tokens(n, 512, 500 + i) for i, n in enumerate(lengths)]
    schedule = eu.mixed(lengths, seed=4, max_live=4)
    lines, wanted = [], []
    for step, (entries, ends) in enumerate(schedule):
        rec = {"step": step, "entries": [], "end": [f"r{i}" for i in ends]}
        for i, a, b in entries:
            want = [k for k in range(b - a) if (a + k) % 3 != 1]        # not every place
            rec["entries"].append({"id": f"r{i}", "tokens": prompts[i][a:b], "want": want})
            wanted.append((step, i, [a + k for k in want]))
        lines.append(json.dumps(rec))
    out_dir = tmp_path / "out"
    proc = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(eu.peak_tokens(lengths, schedule, 64))],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == [w for s in range(len(schedule)) for w in ("done", str(s))]
    expect = [oracle.logits(p) for p in prompts]
    tol = 1e-4 if dtype == "float32" else 2.5e-2
    by_step = {}
    for step, i, places in wanted:
        by_step.setdefault(step, []).append((i, places))
    for step, items in by_step.items():
        rows = sum(len(p) for _, p in items)
        path = out_dir / f"{step}.f32"
        if rows == 0:
            assert not path.exists()
            continue
        data = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(rows, 512))
        r = 0
        for i, places in items:
            if places:
                err = eu.rel_err(data[r:r + len(places)], expect[i][places])
                assert err < tol, f"step {step} request {i}: {err:.3e}"
            r += len(places)


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
