"""Random-weights mode: write a model folder (config.json, model.safetensors)
from a configuration and a seed.

The reference has no such mode (its tests build identity matrices by hand,
/root/reference/src/transformer/hybrid_attn.zig:1108-1170); this one draws every
tensor the model's parts ask for, in the order the spec lists them, from one
seeded generator, so a folder is reproducible from (configuration, seed,
options) alone.

    python -m zig_ai_amd.weights.random_init --config cfg.json --seed 0 --out DIR
"""

from __future__ import annotations

import argparse
import json
import os
from typing import Any, Mapping, Optional

import torch

from ..config import config_from_dict
from .loader import expected_tensors
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def random_tensors(spec, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                   norm_init: str = "ones", role_std: Optional[Mapping[str, float]] = None):
    """Tensors by canonical checkpoint name.

    ``matrix`` / ``table`` / ``bias`` / ``filter`` tensors are N(0, std) (``role_std``
    overrides the deviation per role or per name suffix); norm weights are 1
    (``norm_init="ones"``), N(0, std) (``"normal"``) or 1 + N(0, std)
    (``"around_one"``).  Values are drawn in 32-bit and rounded to ``dtype``.
    """
    if norm_init not in ("ones", "normal", "around_one"):
        raise ValueError(f"norm_init must be ones, normal or around_one, got {norm_init!r}")
    role_std = dict(role_std or {})
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    out = {}
    for exp in expected_tensors(spec):
        name = exp.names[0]
        if name in out:
            continue
        shape = exp.rule.stored_shape or exp.rule.shapes[0]
        dev = role_std.get(exp.rule.role, std)
        for suffix, value in role_std.items():
            if "." in suffix and name.endswith(suffix):
                dev = value
        if exp.rule.role == "norm":
            if norm_init == "ones":
                t = torch.ones(shape, dtype=torch.float32)
            else:
                t = torch.empty(shape, dtype=torch.float32).normal_(0.0, dev, generator=gen)
                if norm_init == "around_one":
                    t += 1.0
        else:
            t = torch.empty(shape, dtype=torch.float32).normal_(0.0, dev, generator=gen)
        out[name] = t.to(dtype)
    return out


def write_random_model(config: Any, out_dir: str, seed: int, dtype: torch.dtype = torch.bfloat16,
                       std: float = 0.02, norm_init: str = "ones",
                       role_std: Optional[Mapping[str, float]] = None) -> str:
    """``config``: a typed configuration or a config.json dictionary."""
    if isinstance(config, Mapping):
        config_dict = dict(config)
        config = config_from_dict(config_dict)
    else:
        config_dict = config.to_dict()
    spec = config.to_spec()
    os.makedirs(out_dir, exist_ok=True)
    tensors = random_tensors(spec, seed, dtype, std, norm_init, role_std)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": str(seed)})
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_dict, f, indent=2)
    return out_dir


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--config", required=True, help="a config.json to take the sizes from")
    ap.add_argument("--out", required=True, help="folder to write")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--dtype", choices=sorted(_DTYPES), default="bfloat16")
    ap.add_argument("--std", type=float, default=0.02)
    ap.add_argument("--norm-init", choices=["ones", "normal", "around_one"], default="ones")
    args = ap.parse_args(argv)
    with open(args.config, "r", encoding="utf-8") as f:
        data = json.load(f)
    write_random_model(data, args.out, args.seed, _DTYPES[args.dtype], args.std, args.norm_init)
    print(f"wrote {args.out}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
