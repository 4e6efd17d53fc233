"""Command line in the manner of the reference's
(/root/reference/src/main.zig:177-319): the same option names with the same
meanings and defaults where the reference has them, the rest dropped with the
subsystems they belonged to (quantisation, offload, speculative decoding, chat
templates), and a few of this engine's own.

    python -m zig_ai_amd -m MODEL_DIR --prompt "12 7 99" -n 32 --temperature 0

``--prompt`` is text when the model folder holds a ``tokenizer.json`` (and the
``tokenizers`` package is there), otherwise token ids separated by spaces or
commas; ``--prompt-ids`` is always ids.
"""

from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="zig-ai", description="LFM2 inference on one MI355X")
    ap.add_argument("-m", "--model", default=None, help="model folder (config.json + safetensors)")
    ap.add_argument("--random-weights", action="store_true",
                    help="no checkpoint: draw weights N(0, 0.02) for --config (or the config.json "
                         "in --model) into a temporary model folder")
    ap.add_argument("--config", default=None, help="a config.json, for --random-weights")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of --random-weights")
    ap.add_argument("--prompt", default=None, help="prompt text, or token ids without a tokenizer")
    ap.add_argument("--prompt-ids", default=None, help="prompt as token ids: \"5 17 3\" or \"5,17,3\"")
    ap.add_argument("--prompt-file", default=None,
                    help="JSON file with a list of prompts, each a list of token ids")
    ap.add_argument("-n", "--max-tokens", type=int, default=128, help="most new tokens (default 128)")
    ap.add_argument("--temperature", type=float, default=1.0, help="default 1.0; <= 0 is greedy")
    ap.add_argument("--top-k", type=int, default=0, help="default 0 = off")
    ap.add_argument("--top-p", type=float, default=1.0, help="default 1.0 = off")
    ap.add_argument("--repetition-penalty", type=float, default=1.0, help="default 1.0 = off")
    ap.add_argument("--seed", type=int, default=42, help="seed of the sampling streams (default 42)")
    ap.add_argument("-b", "--batch-size", type=int, default=2048,
                    help="token budget of one step (default 2048)")
    ap.add_argument("-ub", "--ubatch-size", type=int, default=2048,
                    help="largest portion of one prompt in a step (default 2048, the step's "
                         "whole budget; the reference's own default of 512 reads every weight "
                         "four times per 2,048 prompt tokens: 8.5 ms instead of 5.0 on the "
                         "LFM2-1.2B shape)")
    ap.add_argument("-np", type=int, default=1, dest="num_parallel",
                    help="run the prompt as this many parallel requests (default 1)")
    ap.add_argument("--backend", choices=["auto", "gpu", "cpu"], default="auto",
                    help="auto and gpu run on the GPU; cpu is refused (there is no CPU path)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None)
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--max-model-len", type=int, default=None,
                    help="longest prompt + generation (default: the model's, at most 8192)")
    ap.add_argument("--eos", type=int, default=None, help="stop token id (default: the config's)")
    ap.add_argument("--reproducible", action="store_true",
                    help="every sum in a fixed order: bitwise the same logits run after run "
                         "(bfloat16 decoding otherwise adds to the residual stream with atomics, "
                         "which is faster and reproducible to rounding only)")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch decode steps kernel by kernel instead of replaying HIP graphs "
                         "(the reference's NOGRAPH)")
    ap.add_argument("--portion-graphs", action="store_true",
                    help="also record steps with prompt portions into HIP graphs, from the second "
                         "time a shape (tokens per request, table width) is seen")
    ap.add_argument("--dump-logits", default=None, metavar="DIR",
                    help="write the logits every token is drawn from to DIR/<step>.f32, "
                         "[rows, vocab] little-endian 32-bit (the reference's DUMP_LOGITS)")
    ap.add_argument("--verbose", action="store_true", help="one line per step on standard error")
    ap.add_argument("--profile", action="store_true",
                    help="prompt and generation throughput on standard error at the end "
                         "(the reference's PERF_STAGE)")
    ap.add_argument("--json", action="store_true", help="print one JSON object instead of text")
    return ap


def parse_ids(text: str) -> List[int]:
    parts = [p for p in re.split(r"[\s,]+", text.strip()) if p]
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise SystemExit(f"not a list of token ids: {text!r}")


def load_tokenizer(model_dir: str):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(path)


def main(argv: Optional[List[str]] = None) -> int:
    """Run the command line; failures the user can act on (no GPU, no such model, a
    bad configuration or checkpoint, a prompt beyond the limits) are one line on
    standard error and exit status 1, with the traceback under --verbose."""
    args = build_parser().parse_args(argv)
    try:
        return run(args)
    except (OSError, ValueError, RuntimeError, MemoryError) as err:
        if args.verbose:
            raise
        print(f"zig-ai: {type(err).__name__}: {err}", file=sys.stderr)
        return 1


def run(args) -> int:
    if args.backend == "cpu":
        print("this engine has no CPU path; use --backend gpu", file=sys.stderr)
        return 2
    scratch = None
    if args.random_weights:
        import tempfile
        from .config import load_config
        from .weights import write_random_model
        source = args.config or args.model
        if source is None:
            print("--random-weights needs --config FILE (or --model with a config.json)",
                  file=sys.stderr)
            return 2
        import torch
        scratch = tempfile.TemporaryDirectory(prefix="zigai_random_")
        store = torch.float32 if args.dtype == "float32" else torch.bfloat16
        write_random_model(load_config(source), scratch.name, seed=args.weights_seed, dtype=store)
        args.model = scratch.name
    if not args.model:
        print("give -m MODEL_DIR (or --random-weights --config FILE)", file=sys.stderr)
        return 2
    tokenizer = load_tokenizer(args.model)
    prompts: List[List[int]]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts = [[int(t) for t in p] for p in json.load(f)]
    elif args.prompt_ids is not None:
        prompts = [parse_ids(args.prompt_ids)]
    elif args.prompt is not None:
        if tokenizer is not None:
            prompts = [tokenizer.encode(args.prompt).ids]
        else:
            prompts = [parse_ids(args.prompt)]
    else:
        print("give --prompt, --prompt-ids or --prompt-file", file=sys.stderr)
        return 2
    prompts = [p for p in prompts for _ in range(max(1, args.num_parallel))]

    from .engine.engine import Engine
    if args.dump_logits:
        os.makedirs(args.dump_logits, exist_ok=True)
    phases = {"prompt_tokens": 0, "prompt_s": 0.0, "decode_tokens": 0, "decode_s": 0.0}

    def on_step(info) -> None:
        plan = info["plan"]
        run = sum(e.count for e in plan)
        decode = all(e.count == 1 and e.start > 0 for e in plan)
        phases["decode_tokens" if decode else "prompt_tokens"] += run
        phases["decode_s" if decode else "prompt_s"] += info["seconds"]
        if args.dump_logits and info["logits"].shape[0]:
            info["logits"].cpu().numpy().astype("<f4").tofile(
                os.path.join(args.dump_logits, f"{info['step']}.f32"))
        if args.verbose:
            print(f"step {info['step']}: {len(plan)} requests, {run} tokens, "
                  f"{len(info['tokens'])} drawn, {info['seconds'] * 1e3:.2f} ms", file=sys.stderr)

    load_start = time.perf_counter()
    engine = Engine(args.model, dtype=args.dtype, page_size=args.page_size,
                    num_pages=args.num_pages, max_num_seqs=args.max_num_seqs,
                    max_num_batched_tokens=args.batch_size, chunk_size=args.ubatch_size,
                    max_model_len=args.max_model_len, use_graphs=not args.no_graph, portion_graphs=args.portion_graphs,
                    reproducible=args.reproducible,
                    on_step=on_step if (args.dump_logits or args.verbose or args.profile) else None)
    load_s = time.perf_counter() - load_start
    start = time.perf_counter()
    outputs = engine.generate(prompts, max_new_tokens=args.max_tokens,
                              temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                              repetition_penalty=args.repetition_penalty, seed=args.seed,
                              eos_token_id=args.eos)
    import torch
    torch.cuda.synchronize()
    total_s = time.perf_counter() - start
    n_new = sum(len(o) for o in outputs)
    if args.profile:
        for name in ("prompt", "decode"):
            t, sec = phases[f"{name}_tokens"], phases[f"{name}_s"]
            if t:
                print(f"{name}: {t} tokens in {sec * 1e3:.1f} ms ({t / sec:.1f} tok/s)",
                      file=sys.stderr)
    if scratch is not None:
        scratch.cleanup()
    if args.json:
        print(json.dumps({"outputs": outputs, "load_s": load_s, "generate_s": total_s,
                          "tokens_per_s": n_new / total_s if total_s > 0 else 0.0,
                          "stats": engine.stats()}))
        return 0
    for i, out in enumerate(outputs):
        head = f"[{i}] " if len(outputs) > 1 else ""
        if tokenizer is not None:
            print(head + tokenizer.decode(out))
        print(head + " ".join(str(t) for t in out))
    print(f"load {load_s * 1e3:.0f} ms; {sum(len(p) for p in prompts)} prompt tokens, "
          f"{n_new} new tokens in {total_s * 1e3:.0f} ms ({n_new / total_s:.1f} tok/s)",
          file=sys.stderr)
    return 0
