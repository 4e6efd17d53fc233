"""Interfaces every part obeys, and the registries that map a ``PartSpec.kind``
to its class.

A part knows its own sizes and constants (``params``) and its own tensors; it
never learns which model it is in.  Five families exist:

  mixer              ``forward(x, step, cache) -> y``; declares a cache need
  feed-forward       ``forward(x, step) -> y``
                     (``y`` is ``[T, width]`` or a stack ``[P, T, width]`` of 32-bit
                     partial sums that the following norm adds up)
  norm               ``forward(x) -> y`` and ``add_forward(residual, delta) -> y``
  position encoding  used by mixers: a rotation table, or ``apply(q, k, positions)``
  arrangement        wires a block's parts (it declares their names and families;
                     two norms, a mixer and a feed-forward in the usual block)

plus the embedding and the output head.  All ``forward`` functions take packed
token rows ``[T, width]``: the tokens of every request in the step, one after
the other; ``step`` says where each request's rows begin and what it has cached.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

import torch


# --------------------------------------------------------------- tensor rules
@dataclass(frozen=True)
class TensorRule:
    """What a part expects of one of its tensors.

    ``shapes``: accepted stored shapes; the part receives the tensor reshaped
    to the first.  ``stored_shape``: the shape the random model writer stores
    (the first accepted shape if not given).  ``role`` picks the initialiser and the precision the tensor
    is kept in: ``matrix`` and ``table`` stay in their stored dtype (bfloat16
    stays bfloat16, 32-bit stays 32-bit); ``norm``, ``bias`` and ``filter`` are
    small vectors that are always held in 32-bit.
    """

    shapes: Tuple[Tuple[int, ...], ...]
    role: str = "matrix"
    required: bool = True
    stored_shape: Optional[Tuple[int, ...]] = None


# ---------------------------------------------------------------- cache needs
@dataclass(frozen=True)
class PagedNeed:
    """What a mixer keeps per token, in pages: one or more *planes*, each ``heads``
    vectors of ``width`` elements per token.  Keys and values are two planes of
    ``(num_kv_heads, head_dim)`` (``PagedNeed.kv``); a mixer that keeps one latent
    vector per token has one plane ``(1, width)``; planes may differ in size.  With
    ``window > 0`` only the last ``window`` positions are ever read, so older pages
    can be given back.  ``dtype``: what the planes store (``None``: the run's storage
    type)."""

    planes: Tuple[Tuple[int, int], ...]
    window: int = 0
    dtype: Optional[torch.dtype] = None

    @classmethod
    def kv(cls, num_kv_heads: int, head_dim: int, window: int = 0,
           dtype: Optional[torch.dtype] = None) -> "PagedNeed":
        plane = (int(num_kv_heads), int(head_dim))
        return cls((plane, plane), int(window), dtype)

    @property
    def is_kv(self) -> bool:
        """Two planes of the same size: keys and values, which the attention kernels
        read as one tensor ``[pages, 2, heads, page_size, width]``."""
        return len(self.planes) == 2 and self.planes[0] == self.planes[1]

    def elements_per_token(self) -> int:
        return sum(h * w for h, w in self.planes)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size; 32-bit floats unless ``dtype`` says otherwise.
    A new request's state is ``init`` in every element (zero by default: the cache manager
    fills the slot at admission); a state that starts at a running maximum's ``-inf`` or a
    product's ``1`` says so here.  A state whose elements start at different values stores
    them relative to their start, or treats a request's first portion,
    ``step.ctx_lens_host[i] == 0``, as the start itself."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    init: float = 0.0


# ------------------------------------------------------------------- runtime
@dataclass
class Runtime:
    """Where and how parts compute: the device, and the storage dtype of
    activations (``torch.bfloat16`` for serving, ``torch.float32`` for the
    all-32-bit path)."""

    device: torch.device
    dtype: torch.dtype
    # Whether parts may add their result to the residual stream themselves.  Several
    # ranges of K then add to one element with atomics, in the hardware's order: faster,
    # and reproducible to 32-bit rounding only.  False keeps every sum in a fixed order
    # (bitwise the same result for the same step, run after run).
    stream_additions: bool = True
    # Whether the GEMM library's candidates for a shape of many rows are timed at the
    # shape's first call (the fastest is kept; which one wins can differ from run to
    # run).  None: the process's default (on, unless ZIG_AI_GEMM_TUNE=0).  A runtime that
    # keeps every sum in a fixed order takes the library's first answer.
    library_tuning: Optional[bool] = None

    @property
    def tune(self) -> Optional[bool]:
        """What parts hand to ``ops.linear(..., tune=)``."""
        return False if not self.stream_additions else self.library_tuning


class Part:
    """Base of all parts.  Subclasses set ``kind`` and implement
    ``tensor_rules``; their constructor receives tensors already placed on the
    device in the precision their role prescribes."""

    kind: str = ""

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        return {}

    def __init__(self, params: Mapping[str, Any], tensors: Mapping[str, torch.Tensor],
                 runtime: Runtime):
        self.params = dict(params)
        self.runtime = runtime


class Mixer(Part):
    # A part that sets ``takes_stream`` accepts, in place of the activations ``x``, what
    # ``Norm.deferred`` returned (a norm that has not run yet, which the kernels of
    # ``ops.linear`` / ``ops.linear_swiglu`` can run themselves), and a keyword
    # ``stream``: the 32-bit residual stream, to which it may add its result itself;
    # it then returns ``None``.  What is handed over IS the stream (a norm that has not
    # run reads its rows when the first projection runs): a part must be done with ``x``
    # before it adds anything to ``stream``, or the norm would see the sum.
    takes_stream = False

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        """``PagedNeed``, ``StateNeed`` or ``None``."""
        return None

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    takes_stream = False      # as for Mixer
    opens_with_swiglu = False  # its first product is ``ops.linear_swiglu`` on what it is handed

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def add_forward(self, residual: torch.Tensor, delta: Optional[torch.Tensor],
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``residual`` (32-bit, updated in place) takes ``delta``; the result is
        the norm of the sum.  With ``rows`` only those rows are produced and
        ``residual`` is left alone.  ``delta`` is what a mixer or feed-forward
        returned: ``[T, width]``, or a stack ``[P, T, width]`` of 32-bit partial
        sums whose sum over ``P`` is meant.  Parts with a fused kernel override this."""
        if delta is not None and delta.dim() == 3:
            delta = delta.sum(dim=0)
        if rows is not None:
            h = residual.index_select(0, rows.long())
            if delta is not None:
                h = h + delta.index_select(0, rows.long()).float()
            return self.forward(h)
        if delta is not None:
            residual.add_(delta.float())
        return self.forward(residual)


    def deferred(self, residual: torch.Tensor, rows: Optional[torch.Tensor] = None,
                 swiglu: bool = False):
        """The norm of ``residual`` (of its ``rows``) as something a part with
        ``takes_stream`` accepts in place of activations, without running it now; or
        ``None`` when this norm, or this step, has no such form.  ``swiglu``: the part
        says that its first product is a fused gate|up with its gate (``Part.opens_with_swiglu``),
        for which more row counts have a fused form."""
        return None


class PositionEncoding(Part):
    # Held inside a mixer; the model asks nested parts, too, for ``graph_safe``,
    # ``kernel_sources`` and ``item_granularities``.  ``graph_safe = True`` only if
    # ``apply`` never looks at ``positions`` (or anything of the step) on the host.
    graph_safe = False

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor):
        """Generic path: return encoded ``(q, k)`` of shape ``[T, heads, head_dim]``."""
        raise NotImplementedError


# ---------------------------------------------------------------- registries
_REGISTRIES: Dict[str, Dict[str, Any]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "arrangement": {},
    "embedding": {}, "head": {},
}


def _register(family: str, kind: str, obj: Any) -> Any:
    _REGISTRIES[family][kind] = obj
    return obj


def register_mixer(kind: str, cls: Any) -> Any:
    return _register("mixer", kind, cls)


def register_feed_forward(kind: str, cls: Any) -> Any:
    return _register("feed_forward", kind, cls)


def register_norm(kind: str, cls: Any) -> Any:
    return _register("norm", kind, cls)


def register_position(kind: str, cls: Any) -> Any:
    return _register("position", kind, cls)


def register_arrangement(kind: str, cls: Any) -> Any:
    return _register("arrangement", kind, cls)


def register_embedding(kind: str, cls: Any) -> Any:
    return _register("embedding", kind, cls)


def register_head(kind: str, cls: Any) -> Any:
    return _register("head", kind, cls)


def lookup(family: str, kind: str) -> Any:
    table = _REGISTRIES[family]
    if kind not in table:
        raise KeyError(f"no {family} part named {kind!r}; registered: {', '.join(sorted(table))}")
    return table[kind]
