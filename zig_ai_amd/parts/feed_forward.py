"""Dense SwiGLU feed-forward: ``(silu(x Wg^T) * (x Wu^T)) Wd^T`` without biases
(/root/reference/src/transformer/ffn.zig:19-33).  Gate and up weights are fused
into one ``[2I, H]`` matrix at load so the input is read once.  The result may be
a stack of partial sums (see ``Norm.add_forward``)."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import FeedForward, Runtime, TensorRule, register_feed_forward


def fuse_rows(*mats: torch.Tensor) -> torch.Tensor:
    """Stack weight matrices along the output dimension; mixed precisions are
    widened to 32-bit rather than narrowed."""
    if len({m.dtype for m in mats}) > 1:
        mats = tuple(m.float() for m in mats)
    return torch.cat(mats, dim=0).contiguous()


class SwiGLU(FeedForward):
    kind = "swiglu"
    graph_safe = True
    takes_stream = True
    opens_with_swiglu = True
    kernel_sources = ("gemm", "gemm_rows64", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I = int(params["hidden_size"]), int(params["intermediate_size"])
        return {"gate.weight": TensorRule(((I, H),)), "up.weight": TensorRule(((I, H),)),
                "down.weight": TensorRule(((H, I),))}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.gate_up = fuse_rows(tensors["gate.weight"], tensors["up.weight"])
        self.down = tensors["down.weight"]
        ops.check_projection_weight(self.gate_up, "feed_forward gate_up")
        ops.check_projection_weight(self.down, "feed_forward down")

    def forward(self, x, step=None, stream: Optional[torch.Tensor] = None):
        bf16 = x.dtype == torch.bfloat16 and self.gate_up.dtype == torch.bfloat16
        if bf16 and x.shape[0] <= 16 and x.shape[1] <= 8192:
            # a decode batch: the gate is applied to the projection's accumulators
            a = ops.linear_swiglu(x, self.gate_up)
        elif bf16 and isinstance(x, ops.NormedRows) and ops.rows64_swiglu_fusable(*x.shape):
            # a step beyond 16 rows whose norm has not run: norm, product and gate in one kernel
            a = ops.linear_swiglu(x, self.gate_up)
        else:
            if isinstance(x, ops.NormedRows):
                x = x.materialise()
            a = ops.swiglu(ops.linear(x, self.gate_up, tune=self.runtime.tune))
        return ops.linear(a, self.down, partial_ok=True, accumulate=stream, tune=self.runtime.tune)


register_feed_forward(SwiGLU.kind, SwiGLU)
