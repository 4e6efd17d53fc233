"""The ShortConv mixer as a part: ``in_proj -> (B, C, x)``, ``u = B * x``, a
causal depth-wise convolution of ``kernel_size`` taps over the request's own
inputs (the last ones carried in a fixed-size state slot), ``y = C * conv(u)``,
``out_proj``.  Biases on the three linear/conv maps when ``bias`` is set and the
checkpoint holds them.

The carried-state mechanics follow the reference's convolution
(/root/reference/src/transformer/short_conv.zig:188-225: taps over [state rows;
new rows], state <- last rows); the order project-gate-convolve-gate-project is
the model's definition, which the reference's layer does not follow
(short_conv.zig:174-277 convolves first and gates with SiLU).
"""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, Runtime, StateNeed, TensorRule, register_mixer


class ShortConv(Mixer):
    kind = "short_conv"
    graph_safe = True
    takes_stream = True
    kernel_sources = ("gemm", "gemm_rows64", "shortconv")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, L = int(params["hidden_size"]), int(params["kernel_size"])
        rules = {"in_proj.weight": TensorRule(((3 * H, H),)),
                 "conv.weight": TensorRule(((H, L), (H, 1, L)), role="filter",
                                           stored_shape=(H, 1, L)),
                 "out_proj.weight": TensorRule(((H, H),))}
        if params.get("bias"):
            rules["conv.bias"] = TensorRule(((H,),), role="bias")
            # the projections' biases are used when the checkpoint has them
            rules["in_proj.bias"] = TensorRule(((3 * H,),), role="bias", required=False)
            rules["out_proj.bias"] = TensorRule(((H,),), role="bias", required=False)
        return rules

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        return StateNeed((int(params["hidden_size"]), int(params["kernel_size"])))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.hidden = int(params["hidden_size"])
        self.kernel_size = int(params["kernel_size"])
        if self.kernel_size > 8:
            raise ValueError(f"conv kernel_size {self.kernel_size} exceeds the kernel's limit of 8")
        self.w_in = tensors["in_proj.weight"]
        self.w_out = tensors["out_proj.weight"]
        # the kernel takes the filter tap by tap, [L, hidden]
        self.w_conv = tensors["conv.weight"].reshape(self.hidden, self.kernel_size).t().contiguous()
        self.b_in = tensors.get("in_proj.bias")
        self.b_conv = tensors.get("conv.bias")
        self.b_out = tensors.get("out_proj.bias")
        ops.check_projection_weight(self.w_in, "short_conv w_in")
        ops.check_projection_weight(self.w_out, "short_conv w_out")

    def forward(self, x, step, cache, stream: Optional[torch.Tensor] = None):
        if step.n_tokens == step.n_seqs and self.b_in is None \
                and ops.gated_conv_fusable(x, self.w_in, self.w_conv):
            # a decode batch, one token a request: norm, in_proj and convolution in one kernel
            y = ops.in_proj_gated_conv(x, self.w_in, self.w_conv, self.b_conv, cache.state,
                                       step.slot_id)
        else:
            z = ops.linear(x, self.w_in, self.b_in, tune=self.runtime.tune)
            y = ops.short_conv(z, self.w_conv, self.b_conv, cache.state, step.token_seq,
                               step.seq_start, step.slot_id)
        return ops.linear(y, self.w_out, self.b_out, partial_ok=True, accumulate=stream,
                          tune=self.runtime.tune)


register_mixer(ShortConv.kind, ShortConv)
