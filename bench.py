"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Default run: the layer sizes of the LFM2-1.2B shape (16 layers, hidden 2048, vocabulary 65,536)
with random bfloat16 weights N(0, 0.02), a batch of 8 requests, each prefilled
with 2,048 synthetic tokens and decoded from there (context 4,096).  A step is
one decode step of the whole batch through the engine's own step function and
greedy sampler.  Prints ONE JSON line: decoded tokens per second as ``value``,
a 2,048-token prefill under ``prefill``, the decode step against the HBM
roofline under ``roofline``, and batch 1 / batch 64 decoding under ``points``.
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
        for part in (b.mixer_norm, b.mixer, b.feed_forward_norm, b.feed_forward):
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
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points")
    ap.add_argument("--phase", choices=["all", "prefill", "decode"], default="all",
                    help="measure only one phase (for profiling); the JSON line then holds "
                         "only that phase")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    from zig_ai_amd.engine import DecoderModel, ModelRunner, StepEntry
    from zig_ai_amd.kernels import ops

    torch.cuda.set_device(0)
    cfg = dict(LFM2_1_2B)
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None and args.layers < full_layers:
        cfg["num_hidden_layers"] = args.layers
        cfg["layer_types"] = cfg["layer_types"][:args.layers]
    model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16")
    vocab = cfg["vocab_size"]
    page = 16
    gen = torch.Generator().manual_seed(1234)

    def tokens(n):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    def decode_run(batch, prompt_len, steps, warmup):
        """Prefill ``batch`` requests, then time ``steps`` decode steps."""
        need = batch * ((prompt_len + steps + warmup + 2 + page - 1) // page + 1)
        runner = ModelRunner(model, page_size=page, num_pages=need, num_slots=batch)
        last = []
        for r in range(batch):
            runner.admit(r)
            logits = runner.step([StepEntry(r, tokens(prompt_len), [prompt_len - 1])])
            last.append(int(ops.argmax(logits)[0]))

        def one(cur):
            logits = runner.step([StepEntry(r, [cur[r]], [0]) for r in range(batch)])
            return ops.argmax(logits).tolist()

        for _ in range(warmup):
            last = one(last)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            last = one(last)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx_mid = prompt_len + warmup + steps / 2.0
        for r in range(batch):
            runner.release(r)
        del runner
        torch.cuda.empty_cache()
        return dt, ctx_mid

    # ---- prefill of 2,048 tokens, one request, one step
    T = 2048
    if args.phase == "decode":
        dt, ctx_mid = decode_run(args.batch, args.prompt_len, args.steps, args.warmup)
        print(json.dumps({"phase": "decode", "batch": args.batch, "steps": args.steps,
                          "ms_per_step": dt / args.steps * 1e3,
                          "value": args.batch * args.steps / dt, "unit": "tokens/s"}), flush=True)
        return 0
    runner = ModelRunner(model, page_size=page, num_pages=4 * (T // page + 1), num_slots=4)
    for r in range(2):                                  # warm-up
        runner.admit(("w", r))
        runner.step([StepEntry(("w", r), tokens(T), [T - 1])])
        runner.release(("w", r))
    torch.cuda.synchronize()
    reps = 3
    t0 = time.perf_counter()
    for r in range(reps):
        runner.admit(("p", r))
        runner.step([StepEntry(("p", r), tokens(T), [T - 1])])
        runner.release(("p", r))
    torch.cuda.synchronize()
    prefill_s = (time.perf_counter() - t0) / reps
    del runner
    torch.cuda.empty_cache()
    n_attn = sum(1 for k in cfg["layer_types"] if k != "conv")
    qdim = cfg["num_attention_heads"] * (cfg["hidden_size"] // cfg["num_attention_heads"])
    prefill_flops = 2.0 * T * matmul_params(model) + n_attn * 2.0 * T * T * qdim \
        + 2.0 * vocab * cfg["hidden_size"]
    prefill = {"value": T / prefill_s, "tokens": T, "ms": prefill_s * 1e3,
               "frac": prefill_flops / prefill_s / PEAK_FLOPS["bf16"]}
    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill", **prefill}), flush=True)
        return 0

    # ---- the headline: batch 8 decoding from a 2,048-token context
    dt, ctx_mid = decode_run(args.batch, args.prompt_len, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    hd = cfg["hidden_size"] // cfg["num_attention_heads"]
    kv_bytes_per_token = n_attn * 2 * cfg["num_key_value_heads"] * hd * 2
    step_bytes = count_bytes(model) + args.batch * kv_bytes_per_token * ctx_mid
    achieved = step_bytes / (dt / args.steps)
    roofline = {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_BYTES_PER_S / 1e9,
                "unit": "GB/s", "frac": achieved / HBM_BYTES_PER_S}

    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps = max(16, args.steps // 2)
            d, _ = decode_run(b, args.prompt_len, steps, 4)
            points[f"decode_b{b}"] = b * steps / d

    line = {
        "metric": "decode tok/s @ batch 8 (LFM2-1.2B shape, context 2048 prompt + decode)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic token ids uniform over the vocabulary; random weights N(0, 0.02)",
        "config": {
            "model": "LFM2-1.2B shape", "global_batch": args.batch, "seq_len": 4096,
            "prompt_len": args.prompt_len, "parallelism": "single GPU",
            "layers": cfg["num_hidden_layers"], "layers_of_config": full_layers,
            "attention_layers": n_attn, "hidden_size": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": hd, "ffn_width": model.config.intermediate_size, "vocab": vocab,
            "conv_L_cache": cfg["conv_L_cache"], "rope_theta": cfg["rope_theta"],
            "norm_eps": cfg["norm_eps"], "tied_embeddings": cfg["tie_embedding"],
            "page_size": page, "weights_GB": count_bytes(model) / 1e9,
        },
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
