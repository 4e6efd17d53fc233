"""Architecture-independent description of a decoder: which parts make up each
layer, with which constants, which checkpoint tensors feed them, and in which
order the layers run.

An architecture's typed configuration (for instance ``Lfm2Config``) translates
itself into a ``ModelSpec``; everything below the configuration (loader, model
assembly, cache manager, step function) reads only the spec.  A spec can also
be written by hand, which is how tests assemble models out of toy parts.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A configuration is missing a key, has a wrong type, or is inconsistent."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: a registry key, its constants, and its tensors.

    ``tensors`` maps the part's local tensor names to the checkpoint names that
    may hold them (first name is the canonical one, used when writing).
    """

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    tensors: Mapping[str, Tuple[str, ...]] = field(default_factory=dict)

    def with_params(self, **extra: Any) -> "PartSpec":
        merged = dict(self.params)
        merged.update(extra)
        return PartSpec(self.kind, merged, self.tensors)


@dataclass(frozen=True)
class LayerSpec:
    """A decoder block: its parts by name, and the name of the arrangement that wires
    them together.  The arrangement says which names it has and of which family each
    is (``slots``); the usual block has a mixer, a feed-forward and a norm before each
    (``LayerSpec.pre_norm``), another may have four norms, no feed-forward, or two
    mixers."""

    parts: Mapping[str, PartSpec]
    arrangement: str = "pre_norm_residual"

    @classmethod
    def pre_norm(cls, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                 feed_forward_norm: PartSpec, arrangement: str = "pre_norm_residual") -> "LayerSpec":
        return cls({"mixer_norm": mixer_norm, "mixer": mixer,
                    "feed_forward_norm": feed_forward_norm, "feed_forward": feed_forward},
                   arrangement)

    def __getattr__(self, name: str) -> PartSpec:
        # a part by its name, as an attribute: layer.mixer, layer.feed_forward_norm
        parts = object.__getattribute__(self, "parts")
        if name in parts:
            return parts[name]
        raise AttributeError(name)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers``.  ``cache`` names the cache entry the
    call's mixer uses; two calls with the same ``cache`` share it, and only
    calls with ``writes_cache`` store into it (a reader of another layer's
    cache has ``writes_cache=False``).  ``cache=None`` gives the call an entry
    of its own.
    """

    layer: int
    cache: Optional[int] = None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerCall, ...]
    final_norm: PartSpec
    lm_head: PartSpec
    max_position: int = 0
    ignored_tensors: Tuple[str, ...] = ()    # checkpoint names that may be there and are not read

    def __post_init__(self) -> None:
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        if not self.schedule:
            raise ConfigError("the run order is empty")
        for call in self.schedule:
            if not 0 <= call.layer < len(self.layers):
                raise ConfigError(
                    f"run order names layer {call.layer}, but there are {len(self.layers)} layers")

    def resolved_schedule(self) -> Tuple[LayerCall, ...]:
        """The run order with every ``cache=None`` replaced by a fresh id."""
        used = {c.cache for c in self.schedule if c.cache is not None}
        out = []
        next_id = 0
        for call in self.schedule:
            if call.cache is None:
                while next_id in used:
                    next_id += 1
                used.add(next_id)
                out.append(LayerCall(call.layer, next_id, call.writes_cache))
            else:
                out.append(call)
        return tuple(out)
