"""Rotary position encoding as a part.

``inv_freq[i] = theta^(-2i / rotary_dim)`` and ``angle = position * inv_freq[i]``
(/root/reference/src/transformer/rope.zig:29-43); the pair rotated by that angle
is ``(i, i + rotary_dim/2)`` for ``pairing="half"`` (what the reference's device
kernel does, /root/reference/src/cuda/layer_kernels.cu:353-365) or ``(2i, 2i+1)``
for ``pairing="adjacent"`` (rope.zig:46-53).  ``rotary_dim < head_dim`` rotates
only the leading elements.  The attention mixer applies the rotation inside its
fused query/key kernel; this part only owns the constants.
"""

from __future__ import annotations

import torch

from .base import PositionEncoding, Runtime, register_position


class RotaryEmbedding(PositionEncoding):
    kind = "rope"
    kernel_sources = ("rope_kv",)
    fused_rotation = True   # the mixer's kernel rotates; ``apply`` is not called
    graph_safe = True       # constants only: nothing of a step is looked at on the host

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        self.theta = float(params["theta"])
        self.pairing = str(params.get("pairing", "half"))
        if self.pairing not in ("half", "adjacent"):
            raise ValueError(f"rope pairing must be half or adjacent, got {self.pairing!r}")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim "
                             f"{self.head_dim}")
        i = torch.arange(0, self.rotary_dim // 2, dtype=torch.float64)
        inv = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64),
                              2.0 * i / self.rotary_dim)
        self.inv_freq = inv.to(torch.float32).to(runtime.device)


register_position(RotaryEmbedding.kind, RotaryEmbedding)
