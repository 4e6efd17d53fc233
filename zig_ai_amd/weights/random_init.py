"""Random-weights mode: write a model folder (config.json, model.safetensors)
from a configuration and a seed.

The reference has no such mode (its tests build identity matrices by hand,
/root/reference/src/transformer/hybrid_attn.zig:1108-1170).  Here every value is a
function of (seed, tensor name, element index) alone: a counter-based generator
(Philox-4x32-10, the generator of the sampler's streams in csrc/host.cpp) keyed by
a digest of seed and name, with the element index as its counter.  So a tensor does
not change when another is added, removed or drawn first, and the same tensor comes
out whether it is drawn here, on the CPU, for a folder, or on the GPU for a benchmark
(``DecoderModel.from_random``): the integer stream is identical, and the normal
deviates are made from it in double precision before they are rounded (two
libraries' logarithms and cosines may differ in the last place of a double, which
survives the rounding to 32-bit about once in 10^9 values).

    python -m zig_ai_amd.weights.random_init --config cfg.json --seed 0 --out DIR
"""

from __future__ import annotations

import argparse
import hashlib
import json
import math
import os
from typing import Any, Mapping, Optional, Tuple

import torch

from ..config import config_from_dict
from .loader import expected_tensors
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}

_MASK = 0xFFFFFFFF
_PHILOX_M0, _PHILOX_M1 = 0xD2511F53, 0xCD9E8D57
_PHILOX_W0, _PHILOX_W1 = 0x9E3779B9, 0xBB67AE85


def tensor_key(seed: int, name: str) -> Tuple[int, int]:
    """The generator's 64-bit key for one tensor: the first eight bytes of
    SHA-256("<seed>:<name>")."""
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[0:4], "little"), int.from_bytes(digest[4:8], "little")


def _philox(counter: torch.Tensor, key: Tuple[int, int]):
    """Philox-4x32-10 on counters (counter, 0, 0, 0): four 32-bit words per counter, as
    int64 tensors (products of two 32-bit words wrap in 64 bits, which keeps the low 64
    bits, all that is used)."""
    c0, c1 = counter & _MASK, (counter >> 32) & _MASK
    c2 = torch.zeros_like(counter)
    c3 = torch.zeros_like(counter)
    k0, k1 = key
    for _ in range(10):
        p0 = c0 * _PHILOX_M0
        p1 = c2 * _PHILOX_M1
        hi0, lo0 = (p0 >> 32) & _MASK, p0 & _MASK
        hi1, lo1 = (p1 >> 32) & _MASK, p1 & _MASK
        c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
        k0, k1 = (k0 + _PHILOX_W0) & _MASK, (k1 + _PHILOX_W1) & _MASK
    return c0, c1, c2, c3


def keyed_normal(seed: int, name: str, numel: int, device="cpu",
                 chunk: int = 1 << 24) -> torch.Tensor:
    """``numel`` standard normal deviates (32-bit) for the tensor ``name``: element ``i``
    depends on (seed, name, i) only.  Counter ``i // 4`` yields four words; words (0, 1)
    and (2, 3) each make two deviates by Box-Muller,
    ``sqrt(-2 ln u) * (cos, sin)(2 pi v)`` with ``u = (w + 1) / 2^32``, ``v = w' / 2^32``."""
    key = tensor_key(seed, name)
    out = torch.empty((numel,), dtype=torch.float32, device=device)
    for start in range(0, numel, chunk):                 # (bounded temporaries)
        stop = min(numel, start + chunk)
        first, last = start // 4, (stop + 3) // 4
        counter = torch.arange(first, last, dtype=torch.int64, device=device)
        w = _philox(counter, key)
        parts = []
        for a, b in ((w[0], w[1]), (w[2], w[3])):
            u = (a.to(torch.float64) + 1.0) / 4294967296.0
            v = b.to(torch.float64) / 4294967296.0
            r = torch.sqrt(-2.0 * torch.log(u))
            parts += [r * torch.cos(2.0 * math.pi * v), r * torch.sin(2.0 * math.pi * v)]
        four = torch.stack(parts, dim=1).reshape(-1)      # element 4c + j is word pair j // 2
        out[start:stop] = four[start - 4 * first: stop - 4 * first].to(torch.float32)
    return out


def random_tensor(seed: int, name: str, shape, role: str, dtype: torch.dtype, std: float,
                  norm_init: str, device="cpu", quick: bool = False) -> torch.Tensor:
    """One tensor of a random model: N(0, std) from ``keyed_normal``; norm weights are 1,
    N(0, std) or 1 + N(0, std) by ``norm_init``.  Drawn in 32-bit, rounded to ``dtype``.
    ``quick``: the deviates come from the tensor library's own generator instead, one
    kernel a tensor (seeded by seed and name, but NOT the values a model folder of this
    seed holds): for runs under a profiler's counters, which run every kernel alone, and
    the keyed generator is some hundred small kernels per 16 million values."""
    n = 1
    for d in shape:
        n *= int(d)
    if role == "norm" and norm_init == "ones":
        return torch.ones(tuple(shape), dtype=dtype, device=device)
    if quick:
        g = torch.Generator(device=device)
        g.manual_seed(tensor_key(seed, name)[0] & 0x7FFFFFFF)
        t = torch.empty((n,), dtype=torch.float32, device=device).normal_(generator=g)
        t = t.reshape(tuple(shape)) * float(std)
    else:
        t = keyed_normal(seed, name, n, device).reshape(tuple(shape)) * float(std)
    if role == "norm" and norm_init == "around_one":
        t = t + 1.0
    return t.to(dtype)


def deviation_of(name: str, role: str, std: float, role_std: Mapping[str, float]) -> float:
    dev = role_std.get(role, std)
    for suffix, value in role_std.items():
        if "." in suffix and name.endswith(suffix):
            dev = value
    return dev


def drawing_device():
    """Where tensors are drawn: the GPU when there is one (a model of the LFM2-1.2B shape
    takes minutes on a CPU), else the CPU; the values are the same."""
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() \
        else torch.device("cpu")


def random_tensors(spec, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                   norm_init: str = "ones", role_std: Optional[Mapping[str, float]] = None,
                   device=None):
    """Tensors by canonical checkpoint name.

    ``matrix`` / ``table`` / ``bias`` / ``filter`` tensors are N(0, std) (``role_std``
    overrides the deviation per role or per name suffix); norm weights are 1
    (``norm_init="ones"``), N(0, std) (``"normal"``) or 1 + N(0, std)
    (``"around_one"``).  Values are drawn in 32-bit and rounded to ``dtype``.
    """
    if norm_init not in ("ones", "normal", "around_one"):
        raise ValueError(f"norm_init must be ones, normal or around_one, got {norm_init!r}")
    role_std = dict(role_std or {})
    device = drawing_device() if device is None else device
    out = {}
    for exp in expected_tensors(spec):
        name = exp.names[0]
        if name in out:
            continue
        shape = exp.rule.stored_shape or exp.rule.shapes[0]
        out[name] = random_tensor(seed, name, shape, exp.rule.role, dtype,
                                  deviation_of(name, exp.rule.role, std, role_std), norm_init,
                                  device).cpu()
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
