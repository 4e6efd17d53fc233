"""Arrangements: how two norms, a mixer and a feed-forward form a block.

``pre_norm_residual`` is the reference's decoder block
(/root/reference/src/transformer/hybrid_layer.zig:366-492):

    h = x + mixer(norm1(x));   y = h + feed_forward(norm2(h))

The residual stream is kept in 32-bit.  A block receives the stream and a
``pending`` tensor that has not been added to it yet, and returns the same
pair: every add is then fused with the norm that follows it, including across
the boundary between two blocks.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import register_arrangement


class PreNormResidualBlock:
    kind = "pre_norm_residual"

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.feed_forward_norm = feed_forward_norm
        self.feed_forward = feed_forward

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, torch.Tensor]:
        n1 = self.mixer_norm.add_forward(residual, pending)
        m = self.mixer.forward(n1, step, cache)
        n2 = self.feed_forward_norm.add_forward(residual, m)
        f = self.feed_forward.forward(n2, step)
        return residual, f


register_arrangement(PreNormResidualBlock.kind, PreNormResidualBlock)
