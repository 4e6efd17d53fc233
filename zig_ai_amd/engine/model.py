"""The decoder assembled from a ``ModelSpec``: embedding, blocks in run order,
final norm, output head.  Nothing here is specific to one architecture; the
spec decides which parts make up which layer and in which order layers run.
"""

from __future__ import annotations

from typing import Any, Dict, List, Mapping, Optional, Sequence

import torch

from ..cache.manager import CacheManager, CacheView
from ..config import load_config
from ..config.spec import LayerCall, ModelSpec, PartSpec
from ..kernels import build as kernel_build
from ..kernels import ops
from ..parts import base as parts
from ..weights.loader import load_tensors
from .batch import StepContext

_RUN_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
               "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def run_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine runs in bfloat16 or float32, not {name}")
        return name
    if name not in _RUN_DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")
    return _RUN_DTYPES[name]


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def arrangement_slots(arrangement, layer) -> Dict[str, str]:
    """The names and families of the parts an arrangement wires (its ``slots``), checked
    against the parts the layer's description gives."""
    slots = dict(getattr(arrangement, "slots", None) or {})
    if not slots:
        raise ValueError(f"arrangement {layer.arrangement!r} declares no parts (``slots``)")
    missing = [n for n in slots if n not in layer.parts]
    unknown = [n for n in layer.parts if n not in slots]
    if missing or unknown:
        raise ValueError(f"arrangement {layer.arrangement!r} wires {sorted(slots)}; the layer "
                         f"lacks {missing} and has {unknown} besides")
    return slots


def walk_parts(part):
    """``part`` and every part nested in it (an attribute that is itself a part, as the
    position encoding inside an attention mixer), at any depth."""
    seen, todo = set(), [part]
    while todo:
        p = todo.pop()
        if id(p) in seen:
            continue
        seen.add(id(p))
        yield p
        for v in getattr(p, "__dict__", {}).values():
            if isinstance(v, parts.Part):
                todo.append(v)
            elif isinstance(v, (list, tuple)):
                todo.extend(e for e in v if isinstance(e, parts.Part))
            elif isinstance(v, dict):
                todo.extend(e for e in v.values() if isinstance(e, parts.Part))


class DecoderModel:
    def __init__(self, spec: ModelSpec, tensors: Mapping[Any, Mapping[str, torch.Tensor]],
                 runtime: parts.Runtime):
        self.spec = spec
        self.runtime = runtime

        def make(family: str, part: PartSpec, owner):
            cls = parts.lookup(family, part.kind)
            return cls(part.params, dict(tensors.get(owner, {})), runtime)

        sources = set()

        def note(part) -> None:
            for p in walk_parts(part):
                sources.update(getattr(p, "kernel_sources", ()))

        self.embedding = make("embedding", spec.embedding, ("embedding",))
        note(self.embedding)
        self.blocks = []
        self.mixer_slots: List[List[str]] = []      # per layer: the names of its mixers
        for i, layer in enumerate(spec.layers):
            arrangement = parts.lookup("arrangement", layer.arrangement)
            slots = arrangement_slots(arrangement, layer)
            built = {name: make(family, layer.parts[name], ("layer", i, name))
                     for name, family in slots.items()}
            for p in built.values():
                note(p)
            self.blocks.append(arrangement(built))
            self.mixer_slots.append([n for n, family in slots.items() if family == "mixer"])
        self.final_norm = make("norm", spec.final_norm, ("final_norm",))
        self.head = make("head", spec.lm_head, ("lm_head",))
        note(self.final_norm)
        note(self.head)
        if getattr(self.head, "tied", False):
            self.head.weight = self.embedding.weight     # the same memory, not a copy
        if getattr(self.head, "weight", None) is None:
            raise ValueError("the output head has no weight")

        # Cache entries: a run-order entry's mixer uses the entry named by ``call.cache``;
        # a block with several mixers has one entry per mixer, ``(call.cache, name)``.
        self.schedule: Sequence[LayerCall] = spec.resolved_schedule()
        self.cache_needs: Dict[Any, object] = {}
        for call in self.schedule:
            layer = spec.layers[call.layer]
            for key, name in self.cache_keys(call):
                part = layer.parts[name]
                need = parts.lookup("mixer", part.kind).cache_need(part.params)
                if key in self.cache_needs and self.cache_needs[key] != need:
                    raise ValueError(
                        f"run-order entries sharing cache {key} need different caches: "
                        f"{self.cache_needs[key]} and {need}")
                self.cache_needs[key] = need
        writers = {key for c in self.schedule if c.writes_cache for key, _ in self.cache_keys(c)}
        for call in self.schedule:
            for key, _ in self.cache_keys(call):
                if self.cache_needs[key] is not None and key not in writers:
                    raise ValueError(f"cache {key} is read but no run-order entry writes it")
        # (what a part holds inside it, a mixer's position encoding for one, is asked too)
        top = [self.embedding, self.final_norm, self.head]
        for b in self.blocks:
            top += list(b.parts.values())
        every = [q for p in top for q in walk_parts(p)]
        self.item_granularities = sorted({
            g for p in every for g in getattr(p, "item_granularities", ())})
        self.kernel_sources = sorted(sources)
        # A step may be recorded into a HIP graph only if no part looks at the step's
        # numbers on the host while it runs.
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in every)
        # Compile what this model's parts use (and the host library), together, before
        # the first step.
        if self.kernel_sources:
            wanted = list(self.kernel_sources) + ["host"]
            if "gemm" in self.kernel_sources and runtime.dtype == torch.bfloat16:
                wanted.append("blaslt")     # products of many rows go to the GEMM library
            kernel_build.build_all(wanted, jobs=len(wanted))

    # ------------------------------------------------------------- construction
    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device: Optional[torch.device] = None,
                    reproducible: bool = False, library_tuning: Optional[bool] = None):
        """``reproducible``: every sum in a fixed order (see ``Runtime.stream_additions``).
        ``library_tuning``: see ``Runtime.library_tuning``."""
        device = device or require_gpu()
        config = load_config(model_dir)
        spec = config.to_spec()
        rt = parts.Runtime(device=device, dtype=run_dtype(dtype), stream_additions=not reproducible,
                           library_tuning=library_tuning)
        tensors = load_tensors(model_dir, spec, rt.dtype, device)
        model = cls(spec, tensors, rt)
        model.config = config
        return model

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype="bfloat16",
                    device: Optional[torch.device] = None, std: float = 0.02,
                    norm_init: str = "ones", reproducible: bool = False,
                    role_std: Optional[Mapping[str, float]] = None,
                    library_tuning: Optional[bool] = None, quick: bool = False):
        """The model that ``write_random_model(config, folder, seed, ...)`` followed by
        ``from_folder`` gives, without the trip through a file: every tensor is drawn on the
        device by the same keyed generator (a value depends on seed, tensor name and element
        index only) and kept as the loader would keep it.  ``config`` is a typed
        configuration or a config.json dictionary.  ``quick``: see ``random_tensor`` (other
        values than the folder's, drawn with one kernel a tensor)."""
        from ..config import config_from_dict
        from ..weights.loader import expected_tensors, keep_dtype
        from ..weights.random_init import deviation_of, random_tensor
        device = device or require_gpu()
        if isinstance(config, Mapping):
            config = config_from_dict(config)
        spec = config.to_spec()
        rt = parts.Runtime(device=device, dtype=run_dtype(dtype), stream_additions=not reproducible,
                           library_tuning=library_tuning)
        tensors: Dict[Any, Dict[str, torch.Tensor]] = {}
        for exp in expected_tensors(spec):
            stored = random_tensor(seed, exp.names[0], exp.rule.stored_shape or exp.rule.shapes[0],
                                   exp.rule.role, rt.dtype,
                                   deviation_of(exp.names[0], exp.rule.role, std, role_std or {}),
                                   norm_init, device, quick=quick)
            kept = keep_dtype(stored.dtype, exp.rule.role, rt.dtype)
            tensors.setdefault(exp.owner, {})[exp.local] = \
                stored.reshape(exp.rule.shapes[0]).to(kept).contiguous()
        model = cls(spec, tensors, rt)
        model.config = config
        return model

    def make_cache(self, page_size: int, num_pages, num_slots: int,
                   scatter_pages: bool = True) -> CacheManager:
        return CacheManager(self.cache_needs, page_size, num_pages, num_slots,
                            device=self.runtime.device, dtype=self.runtime.dtype,
                            scatter_pages=scatter_pages)

    def cache_keys(self, call: LayerCall):
        """``[(cache entry, mixer's name)]`` of one run-order entry."""
        names = self.mixer_slots[call.layer]
        if len(names) == 1:
            return [(call.cache, names[0])]
        return [((call.cache, name), name) for name in names]

    def cache_views(self, cache: CacheManager) -> List[Any]:
        """Per run-order entry what its block's ``forward`` receives as ``cache``: the
        mixer's view, or for a block with several mixers (or none) a dictionary from
        the mixers' names to their views."""
        out = []
        for call in self.schedule:
            keys = self.cache_keys(call)
            if len(keys) == 1 and keys[0][0] == call.cache:
                out.append(cache.view(call.cache, call.writes_cache))
            else:
                out.append({name: cache.view(key, call.writes_cache) for key, name in keys})
        return out

    # ------------------------------------------------------------------ forward
    def forward(self, step: StepContext, views: Sequence[CacheView],
                taps: Optional[List[Dict[str, torch.Tensor]]] = None) -> torch.Tensor:
        """Run the step's tokens through every run-order entry and return 32-bit
        logits ``[R, vocab]`` for ``step.logit_rows``.  ``taps`` (diagnostics, as the
        reference's per-layer dumps, /root/reference/src/main.zig:854-860): a list that
        receives one dictionary for the embedding and one per run-order entry, with
        ``"stream"``, the 32-bit residual stream ``[T, width]`` after it, and whatever the
        entry's parts left under ``step.taps`` (the attention mixer: its queries, the
        keys and values it stored, its output); all copies that later kernels do not
        touch."""
        return self._forward(step, views, taps)

    def _forward(self, step: StepContext, views: Sequence[CacheView],
                 taps: Optional[List[Dict[str, torch.Tensor]]]) -> torch.Tensor:
        residual = self.embedding.forward(step.token_ids)
        pending = None
        if taps is not None:
            taps.append({"stream": residual.clone()})
        for call, view in zip(self.schedule, views):
            step.taps = {} if taps is not None else None
            residual, pending = self.blocks[call.layer].forward(residual, pending, step, view)
            if taps is not None:
                now = residual.clone()
                if pending is not None:
                    now += (pending.sum(dim=0) if pending.dim() == 3 else pending).float()
                step.taps["stream"] = now
                taps.append(step.taps)
        step.taps = None
        if step.n_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32,
                               device=self.runtime.device)
        normed = None
        if pending is None and getattr(self.head, "takes_stream", False):
            normed = self.final_norm.deferred(residual, rows=step.logit_rows)
        if normed is None:
            normed = self.final_norm.add_forward(residual, pending, rows=step.logit_rows)
        return self.head.forward(normed)
