"""RMSNorm as a part.  ``out = x / sqrt(mean(x^2) + eps) * weight`` in 32-bit
(/root/reference/src/transformer/norm.zig:6-33); ``add_forward`` fuses the
residual add that precedes the norm in a pre-norm block."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Norm, Runtime, TensorRule, register_norm


class RMSNorm(Norm):
    kind = "rms_norm"
    graph_safe = True
    kernel_sources = ("norm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        return {"weight": TensorRule(((int(params["width"]),),), role="norm")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.dtype == torch.float32:
            out = ops.add_rmsnorm(x2, None, self.weight, self.eps, self.runtime.dtype,
                                  write_residual=False)
        else:
            out = ops.add_rmsnorm(None, x2, self.weight, self.eps, self.runtime.dtype)
        return out.view(shape)

    def add_forward(self, residual: torch.Tensor, delta: Optional[torch.Tensor],
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.runtime.dtype, rows=rows)

    def deferred(self, residual: torch.Tensor, rows: Optional[torch.Tensor] = None,
                 swiglu: bool = False):
        """``swiglu``: the part that takes the rows starts with a fused gate|up product
        (which also has a form for steps of 17 rows and more, see ``ops.rows64_swiglu_fusable``)."""
        # a decode batch in bfloat16: the projection that follows normalises the rows
        n = residual.shape[0] if rows is None else rows.numel()
        if self.runtime.dtype != torch.bfloat16:
            return None
        if not (ops.normed_rows_fusable(n, self.width)
                or (swiglu and ops.rows64_swiglu_fusable(n, self.width))):
            return None
        return ops.NormedRows(residual, self.weight, self.eps, self.runtime.dtype, rows)


register_norm(RMSNorm.kind, RMSNorm)
