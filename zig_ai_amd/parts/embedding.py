"""Token embedding (row gather into the 32-bit residual stream) and the output
head (a projection to 32-bit logits, optionally sharing the embedding table).
/root/reference/src/transformer/embedding.zig:6-41 (which clamps ids; here an
id outside the table is an error raised before the launch) and
/root/reference/src/loader/gguf_model.zig:47-54 (tied fallback)."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from ..kernels import ops
from .base import Part, Runtime, TensorRule, register_embedding, register_head


class TokenEmbedding(Part):
    kind = "token_embedding"
    graph_safe = True
    kernel_sources = ("norm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        return {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                     role="table")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.weight = tensors["weight"]
        self.vocab_size = int(params["vocab_size"])

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return ops.embed_gather(token_ids, self.weight)


class LinearHead(Part):
    kind = "linear_head"
    graph_safe = True
    takes_stream = True       # ``forward`` accepts a norm that has not run yet
    kernel_sources = ("gemm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        if params.get("tied"):
            return {}
        return {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                     role="table")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.tied = bool(params.get("tied"))
        self.weight = tensors.get("weight")   # the model hands a tied head the embedding table

    def forward(self, x) -> torch.Tensor:
        ops.check_projection_weight(self.weight, "output head")
        return ops.linear(x, self.weight, out_dtype=torch.float32, tune=self.runtime.tune)


register_embedding(TokenEmbedding.kind, TokenEmbedding)
register_head(LinearHead.kind, LinearHead)
