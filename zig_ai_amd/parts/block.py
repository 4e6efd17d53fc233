"""Arrangements: how a block's parts are wired.  An arrangement declares its parts
(``slots``: name -> family; the model builds each from the layer's ``PartSpec`` of that
name and hands them over as a dictionary) and runs them in ``forward``.

``pre_norm_residual`` is the reference's decoder block
(/root/reference/src/transformer/hybrid_layer.zig:366-492):

    h = x + mixer(norm1(x));   y = h + feed_forward(norm2(h))

The residual stream is kept in 32-bit.  A block receives the stream and a
``pending`` tensor that has not been added to it yet, and returns the same
pair: every add is then fused with the norm that follows it, including across
the boundary between two blocks.  Where a part says so (``takes_stream``) the norm
before it is handed over without having run (``Norm.deferred``) and the part may add
its result to the stream itself; nothing is pending after it then.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import register_arrangement


class PreNormResidualBlock:
    kind = "pre_norm_residual"
    slots = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm",
             "feed_forward": "feed_forward"}

    def __init__(self, parts):
        self.parts = dict(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer = parts["mixer"]
        self.feed_forward_norm = parts["feed_forward_norm"]
        self.feed_forward = parts["feed_forward"]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        m = apply_normed(self.mixer_norm, self.mixer, residual, pending, step, cache)
        f = apply_normed(self.feed_forward_norm, self.feed_forward, residual, m, step)
        return residual, f


def apply_normed(norm, part, residual: torch.Tensor, pending: Optional[torch.Tensor], *args):
    """``part(norm(residual + pending))``: what is still to be added to the stream
    afterwards, or ``None`` when the part has added it already."""
    if not getattr(part, "takes_stream", False):
        return part.forward(norm.add_forward(residual, pending), *args)
    x = None
    if pending is None:
        x = norm.deferred(residual, swiglu=True) if getattr(part, "opens_with_swiglu", False) \
            else norm.deferred(residual)
    if x is None:
        x = norm.add_forward(residual, pending)
    runtime = getattr(part, "runtime", None)
    adds = runtime is None or getattr(runtime, "stream_additions", True)
    return part.forward(x, *args, stream=residual if adds else None)


register_arrangement(PreNormResidualBlock.kind, PreNormResidualBlock)
