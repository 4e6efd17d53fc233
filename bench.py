"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --shape 2.6b --prompt-len 6144        # another LFM2 shape, same measurement
    python bench.py --shape 350m --workload serve         # 64 requests through the scheduler

Default run: the layer sizes of the LFM2-1.2B shape (16 layers, hidden 2048, vocabulary 65,536)
with random bfloat16 weights N(0, 0.02), a batch of 8 requests, each prefilled
with 2,048 synthetic tokens and decoded from there (context 4,096).  A step is
one decode step of the whole batch through the engine's own step function and
greedy sampler, issued as generation issues them (the tokens of a step reach the
next one on the device; the host reads them every 8 steps).  Prints ONE JSON line: decoded tokens per second as ``value``,
a 2,048-token prefill under ``prefill``, the decode step against the HBM
roofline under ``roofline``, and batch 1 / batch 64 decoding under ``points`` (tokens per
second) with their step times, bytes and fractions under ``points_detail``, where batch 8
at contexts of 4,096 and 8,192 tokens and batch 64 at 4,096 stand too.  Further keys:
``prefill_chunked_512`` (the same 2,048 tokens in four steps of 512, the reference's
``-ub 512``, /root/reference/src/main.zig:57-61), ``shapes`` (batch 8 decoding and the
2,048-token prefill of the LFM2-350M and LFM2-2.6B layer sizes, the latter at its context
of 8,192), and ``calibration``: what this GPU does at best, measured here (a kernel that
only reads 1 GiB; matrix-core instructions issued back to back), with every fraction also
given against those (``frac_measured``).  ``--phase prefill|decode`` runs that phase alone
for a profiler: no calibration kernels, the GEMM library's first answer for every
shape (no timing of candidates, which allocates, frees and waits inside the first steps),
and weights drawn with one kernel a tensor (other values than the default run's).
The model is ``DecoderModel.from_random(cfg, seed=0)``: the tensors that
``write_random_model(cfg, folder, seed=0)`` stores, drawn on the device.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

LFM2_1_2B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 2048, "num_hidden_layers": 16, "num_attention_heads": 32,
    "num_key_value_heads": 8, "vocab_size": 65536,
    "layer_types": ["conv", "conv", "full_attention", "conv", "conv", "full_attention", "conv",
                    "conv", "full_attention", "conv", "full_attention", "conv", "full_attention",
                    "conv", "full_attention", "conv"],
    "block_ff_dim": 12288, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
    "block_ffn_dim_multiplier": 1.0, "rope_theta": 1000000.0, "norm_eps": 1e-5,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 128000,
}


def _shape(hidden, heads, kv_heads, ff, layers, attention_at):
    cfg = dict(LFM2_1_2B)
    cfg.update(hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads,
               block_ff_dim=ff, num_hidden_layers=layers,
               layer_types=["full_attention" if i in attention_at else "conv"
                            for i in range(layers)])
    return cfg


# the shapes the engine is measured on; the default is the first
SHAPES = {
    "1.2b": LFM2_1_2B,
    "350m": _shape(1024, 16, 8, 6656, 16, (2, 5, 8, 10, 12, 14)),
    "2.6b": _shape(2048, 32, 8, 10752, 30, (2, 6, 10, 14, 18, 21, 24, 27)),
}


def serve(cfg, name, n_requests, new_tokens, portion_graphs=False, chunk_size=None) -> dict:
    """Requests with prompts of 128 to 2,048 tokens through the scheduler, the step
    function and the sampler (temperature 0.7), all admitted at once.  Returns the record."""
    import random
    import tempfile

    import torch
    from zig_ai_amd.config import config_from_dict
    from zig_ai_amd.engine import Engine
    from zig_ai_amd.weights import write_random_model

    rng = random.Random(1)
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(128, 2048))]
               for _ in range(n_requests)]
    with tempfile.TemporaryDirectory(prefix="zigai_bench_") as folder:
        write_random_model(config_from_dict(cfg), folder, seed=0, dtype=torch.bfloat16)
        more = {} if chunk_size is None else {"chunk_size": chunk_size}   # (else the engine's default)
        engine = Engine(folder, dtype="bfloat16", page_size=16, max_num_seqs=64,
                        max_num_batched_tokens=4096, max_model_len=4096,
                        portion_graphs=portion_graphs, **more)
        # warm-up: every kind of step once (more than 16 rows of logits among them),
        # so that no library loads its kernels inside the timed run
        engine.generate([p[:64] for p in prompts[:20]], max_new_tokens=4, temperature=0.7, seed=3,
                        eos_token_id=-1)
        # and the run itself once: the GEMM library's candidates for a shape are timed at
        # the shape's first call (some 10 ms each; a server does that once in its life)
        engine.generate(prompts, max_new_tokens=new_tokens, temperature=0.7, seed=3, eos_token_id=-1)
        torch.cuda.synchronize()
        before = dict(engine.stats())
        t0 = time.perf_counter()
        out = engine.generate(prompts, max_new_tokens=new_tokens, temperature=0.7, seed=3,
                              eos_token_id=-1)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        stats = engine.stats()
        chunk = engine.scheduler.chunk_size
        del engine
        torch.cuda.empty_cache()
    prompt_tokens, generated = sum(len(p) for p in prompts), sum(len(o) for o in out)
    with_prompts = stats["seconds_with_prompts"] - before["seconds_with_prompts"]
    return {
        "workload": "serve", "model": f"LFM2-{name} shape", "requests": n_requests,
        "prompt_tokens": prompt_tokens, "generated_tokens": generated, "seconds": dt,
        "generated_per_s": generated / dt, "tokens_per_s": (prompt_tokens + generated) / dt,
        # steps that held prompt portions (beside decoding requests), and the rest
        "seconds_in_steps_with_prompts": with_prompts,
        "seconds_in_decode_steps": stats["step_seconds"] - before["step_seconds"] - with_prompts,
        "steps": stats["steps"] - before["steps"], "preemptions": stats["preemptions"],
        "dtype": "bf16", "chunk_size": chunk,
        "data": "synthetic token ids; random weights N(0, 0.02)"}


def count_bytes(model):
    """Bytes of every weight a decode step reads once (a tied head reads the
    embedding table once; the embedding gather itself reads a few rows)."""
    seen, total = set(), 0

    def add(t):
        nonlocal total
        if t is not None and t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()

    add(model.head.weight)
    add(model.final_norm.weight)
    for b in model.blocks:
        for part in b.parts.values():
            for v in vars(part).values():
                if hasattr(v, "data_ptr"):
                    add(v)
    return total


def matmul_params(model):
    """Parameters that a token multiplies (everything but the embedding gather)."""
    n = 0
    for b in model.blocks:
        for part in (b.mixer, b.feed_forward):
            for v in vars(part).values():
                if hasattr(v, "dim") and v.dim() == 2 and v.shape[0] > 8:
                    n += v.numel()
    return n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="1.2b",
                    help="layer sizes: LFM2-1.2B (the default run), 350M or 2.6B")
    ap.add_argument("--workload", choices=["steps", "serve"], default="steps",
                    help="steps: decode steps and one prefill (the default run); serve: 64 "
                         "requests with prompts of 128-2048 tokens and 256 new tokens each "
                         "through the scheduler")
    ap.add_argument("--requests", type=int, default=64, help="requests of --workload serve")
    ap.add_argument("--new-tokens", type=int, default=256, help="new tokens per request of "
                    "--workload serve")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points")
    ap.add_argument("--chunk-size", type=int, default=None,
                    help="--workload serve: the longest portion of a prompt in one step "
                         "(default: the engine's own)")
    ap.add_argument("--portion-graphs", action="store_true",
                    help="--workload serve: also record steps with prompt portions")
    ap.add_argument("--phase", choices=["all", "prefill", "decode"], default="all",
                    help="measure only one phase (for profiling); the JSON line then holds "
                         "only that phase")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="--phase prefill: the prompt's length (in steps of 2,048 tokens, or of "
                    "--chunk-size)")
    ap.add_argument("--tuned", action="store_true",
                    help="with --phase: let the GEMM library time its candidates as a plain run "
                         "does (not under a profiler's counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    from zig_ai_amd.kernels import ops

    torch.cuda.set_device(0)
    cfg = dict(SHAPES[args.shape])
    if args.workload == "serve":
        print(json.dumps(serve(cfg, args.shape.upper(), args.requests, args.new_tokens,
                               args.portion_graphs, args.chunk_size)), flush=True)
        return 0
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None and args.layers < full_layers:
        cfg["num_hidden_layers"] = args.layers
        cfg["layer_types"] = cfg["layer_types"][:args.layers]
    page = 16
    gen = torch.Generator().manual_seed(1234)
    profiled = args.phase != "all" and not args.tuned

    def tokens(n, vocab):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    class Measured:
        """One shape's model with what is measured on it."""

        def __init__(self, cfg):
            self.cfg = cfg
            # (a profiled phase takes the library's first answer for every shape, and its
            # weights are drawn with one kernel a tensor: a profiler's counter mode runs
            # every kernel alone, and the keyed generator is some 19,000 small ones)
            self.model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16",
                                                  library_tuning=False if profiled else None,
                                                  quick=profiled)
            self.vocab = cfg["vocab_size"]
            self.n_attn = sum(1 for k in cfg["layer_types"] if k != "conv")
            self.hd = cfg["hidden_size"] // cfg["num_attention_heads"]
            self.kv_bytes_per_token = self.n_attn * 2 * cfg["num_key_value_heads"] * self.hd * 2
            self.weight_bytes = count_bytes(self.model)

        def decode_run(self, batch, prompt_len, steps, warmup):
            """Prefill ``batch`` requests, then time ``steps`` decode steps.  Returns the
            seconds and the mean context length over the timed steps."""
            model, vocab = self.model, self.vocab
            need = batch * ((prompt_len + steps + warmup + 2 + page - 1) // page + 1)
            runner = ModelRunner(model, page_size=page, num_pages=need, num_slots=batch)
            last = []
            for r in range(batch):
                runner.admit(r)
                toks = tokens(prompt_len, vocab)
                for lo in range(0, prompt_len, 2048):            # prompts in steps of 2,048
                    hi = min(prompt_len, lo + 2048)
                    logits = runner.step([StepEntry(r, toks[lo:hi],
                                                    [hi - lo - 1] if hi == prompt_len else [])])
                last.append(int(ops.argmax(logits)[0]))
            requests = list(range(batch))

            greedy = lambda logits, i: ops.argmax(logits)
            pinned = [torch.empty((8 * batch,), dtype=torch.int32, pin_memory=True) for _ in range(2)]

            def run(cur, n):
                """``n`` decode steps the way generation issues them (``Engine``): greedy
                tokens handed from step to step on the device, in runs of 8; the host reads
                a run's tokens, from pinned memory behind an event, once the next run is
                issued."""
                done, device, waiting, turn = 0, None, None, 0
                while done < n:
                    k = min(8, n - done)
                    drawn = runner.decode_steps(requests, cur, k, greedy, device_tokens=device)
                    k = drawn.shape[0]
                    pinned[turn][:k * batch].copy_(drawn.view(-1), non_blocking=True)
                    event = torch.cuda.Event()
                    event.record()
                    if waiting is not None:
                        waiting[0].synchronize()
                        waiting[1].tolist()
                    waiting = (event, pinned[turn][:k * batch])
                    turn ^= 1
                    device, cur = drawn[k - 1], None
                    done += k
                waiting[0].synchronize()
                return waiting[1].view(-1, batch)[-1].tolist()

            last = run(last, warmup)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            last = run(last, steps)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            ctx_mid = prompt_len + warmup + steps / 2.0
            for r in range(batch):
                runner.release(r)
            del runner
            torch.cuda.empty_cache()
            return dt, ctx_mid

        def prefill_flops(self, T):
            cfg = self.cfg
            qdim = cfg["num_attention_heads"] * self.hd
            return 2.0 * T * matmul_params(self.model) + self.n_attn * 2.0 * T * T * qdim \
                + 2.0 * self.vocab * cfg["hidden_size"]

        def prefill_run(self, T, portion, calibration, reps=8, warm=4):
            model, vocab = self.model, self.vocab
            runner = ModelRunner(model, page_size=page, num_pages=4 * (T // page + 1), num_slots=4)

            def one(name):
                runner.admit(name)
                toks = tokens(T, vocab)
                for lo in range(0, T, portion):
                    hi = min(T, lo + portion)
                    runner.step([StepEntry(name, toks[lo:hi], [hi - lo - 1] if hi == T else [])])
                runner.release(name)

            for r in range(warm):                               # warm-up
                one(("w", r))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for r in range(reps):
                one(("p", r))
            torch.cuda.synchronize()
            seconds = (time.perf_counter() - t0) / reps
            del runner
            torch.cuda.empty_cache()
            rate = self.prefill_flops(T) / seconds
            out = {"value": T / seconds, "tokens": T, "ms": seconds * 1e3,
                   "frac": rate / PEAK_FLOPS["bf16"]}
            if calibration:
                out["frac_measured"] = rate / (calibration["mfma_bf16_TFLOPs"] * 1e12)
            return out

        def against_memory(self, batch, seconds_per_step, ctx, calibration):
            """A decode step against the memory it has to read: every weight once and the
            cache of the live requests."""
            step_bytes = self.weight_bytes + batch * self.kv_bytes_per_token * ctx
            rate = step_bytes / seconds_per_step
            out = {"ms_per_step": seconds_per_step * 1e3, "ctx": ctx, "bytes": step_bytes,
                   "achieved_GBps": rate / 1e9, "frac": rate / HBM_BYTES_PER_S}
            if calibration:
                out["frac_measured"] = rate / (calibration["read_GBps"] * 1e9)
            return out

    T = 2048
    main_shape = Measured(cfg)
    ffn_width = main_shape.model.config.intermediate_size
    # ---- one phase alone, for a profiler: nothing else runs
    if args.phase == "decode":
        dt, ctx_mid = main_shape.decode_run(args.batch, args.prompt_len, args.steps, args.warmup)
        print(json.dumps({"phase": "decode", "batch": args.batch, "steps": args.steps,
                          "ms_per_step": dt / args.steps * 1e3,
                          "value": args.batch * args.steps / dt, "unit": "tokens/s"}), flush=True)
        return 0
    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill",
                          **main_shape.prefill_run(args.prefill_tokens, args.chunk_size or T, None)}),
              flush=True)
        return 0

    # ---- what this GPU does at best
    calibration = {"read_GBps": ops.measured_read_bandwidth() / 1e9,
                   "mfma_bf16_TFLOPs": ops.measured_mfma_rate() / 1e12}

    # ---- prefill of 2,048 tokens, one request: in one step, and in four steps of 512
    prefill = main_shape.prefill_run(T, T, calibration)
    prefill_chunked = main_shape.prefill_run(T, 512, calibration)

    # ---- the headline: batch 8 decoding from a 2,048-token context
    dt, ctx_mid = main_shape.decode_run(args.batch, args.prompt_len, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    headline = main_shape.against_memory(args.batch, dt / args.steps, ctx_mid, calibration)
    roofline = {"bound": "hbm", "achieved": headline["achieved_GBps"], "peak": HBM_BYTES_PER_S / 1e9,
                "unit": "GB/s", "frac": headline["frac"], "frac_measured": headline["frac_measured"]}

    points, points_detail, shapes = {}, {}, {}
    if not args.no_points:
        for b in (1, 64):
            steps = max(16, args.steps // 2)
            d, ctx = main_shape.decode_run(b, args.prompt_len, steps, 4)
            points[f"decode_b{b}"] = b * steps / d
            points_detail[f"decode_b{b}"] = main_shape.against_memory(b, d / steps, ctx, calibration)
        # the batch sizes between: the last that this package's kernels for up to 16 rows
        # take, and the steps of 17 to 32 rows
        for b in (16, 24, 32):
            d, ctx = main_shape.decode_run(b, args.prompt_len, 32, 4)
            points_detail[f"decode_b{b}"] = main_shape.against_memory(b, d / 32, ctx, calibration)
        # further contexts (prefilled to there, 16 steps each)
        for b, ctx0 in ((8, 4096), (8, 8192), (64, 4096)):
            d, ctx = main_shape.decode_run(b, ctx0, 16, 4)
            points_detail[f"decode_b{b}_ctx{ctx0}"] = main_shape.against_memory(b, d / 16, ctx, calibration)
        # the other shapes: batch 8 decoding and a 2,048-token prefill each
        if args.shape == "1.2b" and args.layers is None:
            del main_shape.model
            torch.cuda.empty_cache()
            for name, ctx0 in (("350m", 2048), ("2.6b", 8192)):
                other = Measured(dict(SHAPES[name]))
                d, ctx = other.decode_run(8, ctx0, 16, 4)
                detail = other.against_memory(8, d / 16, ctx, calibration)
                detail.update(value=8 * 16 / d, unit="tokens/s", batch=8,
                              layers=other.cfg["num_hidden_layers"],
                              weights_GB=other.weight_bytes / 1e9,
                              prefill=other.prefill_run(T, T, calibration, reps=4, warm=2))
                shapes[name] = detail
                del other
                torch.cuda.empty_cache()
            # and the mixed workload of the 350M shape: 64 requests through the scheduler
            record = serve(dict(SHAPES["350m"]), "350M", 64, 256)
            shapes["350m"]["serve"] = {k: record[k] for k in (
                "requests", "prompt_tokens", "generated_tokens", "seconds", "generated_per_s",
                "tokens_per_s", "seconds_in_steps_with_prompts", "seconds_in_decode_steps", "steps")}

    vocab, hd, n_attn = cfg["vocab_size"], main_shape.hd, main_shape.n_attn
    line = {
        "metric": f"decode tok/s @ batch {args.batch} (LFM2-{args.shape.upper()} shape, context "
                  f"{args.prompt_len} prompt + decode)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic token ids uniform over the vocabulary; random weights N(0, 0.02)",
        "config": {
            "model": f"LFM2-{args.shape.upper()} shape", "global_batch": args.batch,
            # the context the timed steps really reach
            "seq_len": args.prompt_len + args.warmup + args.steps,
            "prompt_len": args.prompt_len, "parallelism": "single GPU",
            "layers": cfg["num_hidden_layers"], "layers_of_config": full_layers,
            "attention_layers": n_attn, "hidden_size": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": hd, "ffn_width": ffn_width, "vocab": vocab,
            "conv_L_cache": cfg["conv_L_cache"], "rope_theta": cfg["rope_theta"],
            "norm_eps": cfg["norm_eps"], "tied_embeddings": cfg["tie_embedding"],
            "page_size": page, "weights_GB": main_shape.weight_bytes / 1e9,
        },
        "prefill": prefill, "roofline": roofline, "points": points,
        "points_detail": points_detail, "prefill_chunked_512": prefill_chunked,
        "shapes": shapes, "calibration": calibration,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
