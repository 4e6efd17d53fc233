"""Loading a model folder's tensors by name against a ``ModelSpec``.

Every part states which tensors it wants (``tensor_rules``) and the spec says
under which checkpoint names they may be stored.  The loader matches the two,
and reports everything that does not fit in ONE error: tensors that are
missing, tensors nothing asked for, wrong shapes and unsupported dtypes.  (The
reference stops at the first absent tensor, ``error.WeightFileNotFound``:
/root/reference/src/transformer/short_conv.zig:492-497, and declares a shape
error it never raises: short_conv.zig:27-30.)

Precision kept on the device:
  * integer tensors become int32;
  * ``matrix`` / ``table`` tensors keep their stored dtype in a bfloat16 run
    (bfloat16 stays bfloat16, a 32-bit tensor stays 32-bit; float16 is widened
    to 32-bit) and are widened to 32-bit in a float32 run;
  * ``norm`` / ``bias`` / ``filter`` tensors are always widened to 32-bit.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Iterator, List, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from ..parts import base as parts_base
from .safetensors_io import Checkpoint, SafetensorsError

Owner = Tuple[Any, ...]

_FLOAT_NAMES = ("BF16", "F16", "F32")
_INT_NAMES = ("I64", "I32", "I16", "I8", "U8")


class WeightError(ValueError):
    """The checkpoint does not fit the model; the message lists every misfit."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)


@dataclass(frozen=True)
class Expected:
    owner: Owner
    local: str
    names: Tuple[str, ...]
    rule: parts_base.TensorRule


def _part_expectations(owner: Owner, family: str, part: PartSpec) -> Iterator[Expected]:
    cls = parts_base.lookup(family, part.kind)
    rules = cls.tensor_rules(part.params)
    for local, rule in rules.items():
        names = tuple(part.tensors.get(local, ()))
        if not names:
            if rule.required:
                raise KeyError(
                    f"part {part.kind!r} at {owner} needs tensor {local!r} but the spec gives "
                    "it no checkpoint name")
            continue
        yield Expected(owner, local, names, rule)
    for key, value in part.params.items():
        if isinstance(value, PartSpec):
            yield from _part_expectations(owner + (key,), "position", value)


def expected_tensors(spec: ModelSpec) -> List[Expected]:
    out: List[Expected] = []
    out += _part_expectations(("embedding",), "embedding", spec.embedding)
    for i, layer in enumerate(spec.layers):
        # the arrangement names the layer's parts and says of which family each is
        slots = getattr(parts_base.lookup("arrangement", layer.arrangement), "slots", {})
        for name, family in slots.items():
            if name not in layer.parts:
                raise KeyError(f"layer {i}: arrangement {layer.arrangement!r} wires a part "
                               f"{name!r} that the layer's description does not give")
            out += _part_expectations(("layer", i, name), family, layer.parts[name])
    out += _part_expectations(("final_norm",), "norm", spec.final_norm)
    out += _part_expectations(("lm_head",), "head", spec.lm_head)
    return out


def keep_dtype(stored: torch.dtype, role: str, run_dtype: torch.dtype) -> torch.dtype:
    """The dtype a tensor has on the device (see the module text)."""
    if not stored.is_floating_point:
        return torch.int32
    if role in ("norm", "bias", "filter"):
        return torch.float32
    if run_dtype == torch.float32:
        return torch.float32
    if stored == torch.bfloat16:
        return torch.bfloat16
    return torch.float32


def load_tensors(model_dir: str, spec: ModelSpec, run_dtype: torch.dtype,
                 device: torch.device | str) -> Dict[Owner, Dict[str, torch.Tensor]]:
    """Return ``{owner: {local name: device tensor}}`` or raise ``WeightError``."""
    try:
        ckpt = Checkpoint(model_dir)
    except SafetensorsError as e:
        raise WeightError(str(e)) from e
    wanted = expected_tensors(spec)
    missing, wrong_shape, wrong_dtype = [], [], []
    chosen: List[Tuple[Expected, str]] = []
    consumed = set()
    for exp in wanted:
        found = next((n for n in exp.names if n in ckpt), None)
        if found is None:
            if exp.rule.required:
                missing.append(exp.names[0])
            continue
        consumed.add(found)
        shape = tuple(ckpt.shape(found))
        if shape not in exp.rule.shapes:
            wrong_shape.append(
                f"{found}: stored {list(shape)}, expected "
                + " or ".join(str(list(s)) for s in exp.rule.shapes))
            continue
        dname = ckpt.dtype_name(found)
        if dname not in _FLOAT_NAMES + _INT_NAMES:
            wrong_dtype.append(f"{found}: {dname}")
            continue
        chosen.append((exp, found))
    unexpected = sorted(n for n in ckpt.names()
                        if n not in consumed and n not in spec.ignored_tensors)
    if missing or unexpected or wrong_shape or wrong_dtype:
        lines = [f"the tensors in {model_dir} do not fit the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shape ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if wrong_dtype:
            lines.append(f"  unsupported dtype ({len(wrong_dtype)}): " + "; ".join(wrong_dtype))
        raise WeightError("\n".join(lines), missing, unexpected, wrong_shape, wrong_dtype)

    out: Dict[Owner, Dict[str, torch.Tensor]] = {}
    for exp, found in chosen:
        try:
            t = ckpt.tensor(found)
        except SafetensorsError as e:
            raise WeightError(str(e)) from e
        t = t.reshape(exp.rule.shapes[0])
        target = keep_dtype(t.dtype, exp.rule.role, run_dtype)
        out.setdefault(exp.owner, {})[exp.local] = t.to(device=device, dtype=target).contiguous()
    return out
