"""Grouped-query attention over a paged cache, as a part.

Per token (/root/reference/src/transformer/hybrid_attn.zig:286-640):
  q, k, v = x Wq^T, x Wk^T, x Wv^T           (one fused projection, optional bias)
  q, k    = per-head RMSNorm(q), RMSNorm(k)  if ``qk_norm``   (371-382)
  q, k    = position encoding(q, k)          (rotary: fused into the same kernel)
  k, v   -> the request's pages
  o       = softmax(q k^T * scale, causal [, window]) v       (553-608)
  y       = o Wo^T

All sizes come from ``params``: ``hidden_size, num_heads, num_kv_heads,
head_dim, qk_norm, norm_eps, window`` (0 = all keys), ``softmax_scale`` (None =
1/sqrt(head_dim)), ``bias`` and ``position`` (a nested position-encoding spec or
None).
"""

from __future__ import annotations

import math
from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import (Mixer, PagedNeed, Runtime, TensorRule, lookup, register_mixer)
from .feed_forward import fuse_rows

# Cutting long contexts pays only when the launch would otherwise leave most of the
# machine idle (decoding few requests, or a portion of a prompt far into a long
# request).  Measured on one MI355X with 8 key/value heads, contexts from 2,048 to
# 131,072 keys and 1 to 64 requests: from 512 workgroups on nothing is gained; below,
# as many ranges as still stay within SPLIT_TARGET workgroups (one decode workgroup of
# eight waves a compute unit) are best or within a few percent of it, all of the same length.
BUSY_WORKGROUPS = 512
SPLIT_TARGET = 256
SPLIT_KEYS_MIN = 512
SPLIT_MAX = 64


def plan_split(n_items: int, num_kv_heads: int, max_keys: int, target: int = SPLIT_TARGET):
    """(keys per range, number of ranges) for one launch; a function of the batch
    shape and of the longest context only.  ``target``: workgroups to reach (the
    kernel for prompt portions runs two workgroups per compute unit and wants 512)."""
    groups = n_items * num_kv_heads
    # (a range of 512 keys is one tile for each of the decode kernel's eight waves; short
    # contexts are cut finer: decoding one request at 512 keys, 4 ranges 0.692 ms a step,
    # none 0.707; at 8,192 keys ranges of 512 0.745, of 256 0.774)
    keys_min = SPLIT_KEYS_MIN if max_keys > 4 * SPLIT_KEYS_MIN else SPLIT_KEYS_MIN // 2
    if groups >= BUSY_WORKGROUPS or max_keys <= 2 * keys_min:
        return 0, 1
    # as many ranges as keep the launch within `target` workgroups (one more range would send
    # part of them into a second round: 12 requests at 2,048 keys, 2 ranges 0.862 ms a step, 3
    # ranges 0.878; 20 requests uncut 1.18, in 2 ranges 1.27)
    wanted = target // groups
    nsplit = min(wanted, max_keys // keys_min, SPLIT_MAX)
    if nsplit <= 1:
        return 0, 1
    keys = ((max_keys + nsplit - 1) // nsplit + 63) // 64 * 64   # a multiple of the key tile
    nsplit = (max_keys + keys - 1) // keys
    return (keys, nsplit) if nsplit > 1 else (0, 1)


class GroupedQueryAttention(Mixer):
    kind = "gqa_attention"
    graph_safe = True
    takes_stream = True
    kernel_sources = ("gemm", "gemm_rows64", "rope_kv", "attention", "norm", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, nh, nkv, d = (int(params[k]) for k in
                         ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        rules = {"q_proj.weight": TensorRule(((nh * d, H),)),
                 "k_proj.weight": TensorRule(((nkv * d, H),)),
                 "v_proj.weight": TensorRule(((nkv * d, H),)),
                 "out_proj.weight": TensorRule(((H, nh * d),))}
        if params.get("qk_norm"):
            rules["q_norm.weight"] = TensorRule(((d,),), role="norm")
            rules["k_norm.weight"] = TensorRule(((d,),), role="norm")
        if params.get("bias"):
            rules["q_proj.bias"] = TensorRule(((nh * d,),), role="bias")
            rules["k_proj.bias"] = TensorRule(((nkv * d,),), role="bias")
            rules["v_proj.bias"] = TensorRule(((nkv * d,),), role="bias")
            rules["out_proj.bias"] = TensorRule(((H,),), role="bias")
        return rules

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        return PagedNeed.kv(int(params["num_kv_heads"]), int(params["head_dim"]),
                            int(params.get("window") or 0))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads do not divide into {self.num_kv_heads} groups")
        self.group = self.num_heads // self.num_kv_heads
        if self.group > ops.ATTENTION_MAX_ROWS:
            raise ValueError(f"{self.group} query heads per key/value head exceed the attention "
                             f"kernel's limit of {ops.ATTENTION_MAX_ROWS}")
        if self.head_dim % 16 or self.head_dim > 256:
            raise ValueError(f"head_dim {self.head_dim} must be a multiple of 16, at most 256")
        # tokens per work item of the two attention kernels
        self.rows_per_item = max(1, ops.ATTENTION_MAX_ROWS // self.group)
        self.mfma_rows_per_item = max(1, ops.ATTENTION_MFMA_ROWS // self.group)
        self.mfma_decode_rows_per_item = max(1, ops.ATTENTION_MFMA_DECODE_ROWS // self.group)
        self.window = int(params.get("window") or 0)
        scale = params.get("softmax_scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        # whether the matrix-core kernels take these sizes (the page size is checked per step)
        self.mfma = ops.attention_mfma_supported(runtime.dtype, self.num_heads,
                                                 self.num_kv_heads, self.head_dim,
                                                 scale=self.scale)
        self.item_granularities = [self.rows_per_item] + (
            [self.mfma_rows_per_item, self.mfma_decode_rows_per_item] if self.mfma else [])
        self.eps = float(params.get("norm_eps", 0.0))
        self.w_qkv = fuse_rows(tensors["q_proj.weight"], tensors["k_proj.weight"],
                               tensors["v_proj.weight"])
        self.w_out = tensors["out_proj.weight"]
        self.b_qkv = self.b_out = None
        if params.get("bias"):
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"],
                                    tensors["v_proj.bias"]]).contiguous()
            self.b_out = tensors["out_proj.bias"]
        self.q_norm = tensors.get("q_norm.weight") if params.get("qk_norm") else None
        self.k_norm = tensors.get("k_norm.weight") if params.get("qk_norm") else None
        pos = params.get("position")
        self.position = None
        if pos is not None:
            self.position = lookup("position", pos.kind)(pos.params, {}, runtime)
        self.fused_rotation = bool(getattr(self.position, "fused_rotation", False))
        # recorded into a graph only if the position encoding, too, never looks at a
        # step's numbers on the host
        self.graph_safe = self.position is None or bool(getattr(self.position, "graph_safe", False))
        # a decode step's norm, rotation and cache write can run inside its attention kernel
        self.rotation_in_attention = (
            self.fused_rotation and runtime.dtype == torch.bfloat16
            and self.position.rotary_dim == self.head_dim and self.position.pairing != "adjacent")
        ops.check_projection_weight(self.w_qkv, "attention w_qkv")
        ops.check_projection_weight(self.w_out, "attention w_out")

    def forward(self, x, step, cache, stream: Optional[torch.Tensor] = None):
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        T = x.shape[0]
        qkv = ops.linear(x, self.w_qkv, self.b_qkv, tune=self.runtime.tune)
        slots = step.slot_mapping[cache.group]
        if self.rotation_in_attention and step.n_tokens == step.n_seqs and cache.writes \
                and ops.decode_rope_fusable(qkv, nh, nkv, d, d, False, cache.kv.shape[3], self.scale):
            # single tokens only: the attention kernel prepares queries, key and value itself
            keys, nsplit = plan_split(step.n_seqs, nkv, step.max_keys)
            # few rows in few ranges: the output projection merges the ranges on its way in
            unmerged = stream is not None and self.b_out is None and ops.merged_rows_pay(T, nsplit)
            o = ops.rope_attention_decode(qkv, step.positions, slots, self.q_norm, self.k_norm,
                                          self.position.inv_freq, cache.kv,
                                          step.block_tables[cache.group], nh, self.eps, self.scale,
                                          self.window, keys, nsplit, combine=not unmerged)
            if getattr(step, "taps", None) is not None:
                # (diagnostics want the queries too: from the kernel the attention replaced)
                q = ops.qk_norm_rope_kv_write(qkv, step.positions, None, self.q_norm, self.k_norm,
                                              self.position.inv_freq, None, nh, nkv, d, d, False,
                                              self.eps, write_kv=False)
                merged = o.materialise() if isinstance(o, ops.MergedRows) else o
                self._leave_taps(step, cache, q, merged.view(T, nh, d))
            if not isinstance(o, ops.MergedRows):
                o = o.view(T, nh * d)
            return ops.linear(o, self.w_out, self.b_out, partial_ok=True, accumulate=stream,
                              tune=self.runtime.tune)
        if self.position is None or self.fused_rotation:
            rot = self.position.rotary_dim if self.position is not None else 0
            q = ops.qk_norm_rope_kv_write(
                qkv, step.positions, slots, self.q_norm, self.k_norm,
                self.position.inv_freq if rot else None, cache.kv, nh, nkv, d, rot,
                bool(rot) and self.position.pairing == "adjacent", self.eps,
                write_kv=cache.writes)
        else:
            # Any other encoding: norm with the norm kernel, encode through the part's own
            # ``apply``, then let the fused kernel store what it is given.  q and k are
            # taken out of the projection's rows and put back by a copy kernel.
            qh = ops.copy_columns(qkv, 0, nh * d)
            kh = ops.copy_columns(qkv, nh * d, nkv * d)
            if self.q_norm is not None:
                qh = ops.add_rmsnorm(None, qh.view(T * nh, d), self.q_norm, self.eps, qkv.dtype)
                kh = ops.add_rmsnorm(None, kh.view(T * nkv, d), self.k_norm, self.eps, qkv.dtype)
            qh, kh = self.position.apply(qh.view(T, nh, d), kh.view(T, nkv, d), step.positions)
            if tuple(qh.shape) != (T, nh, d) or tuple(kh.shape) != (T, nkv, d):
                raise ValueError(f"position encoding {self.position.kind!r} returned "
                                 f"{tuple(qh.shape)} and {tuple(kh.shape)}")
            packed = torch.empty_like(qkv)
            ops.copy_columns(qh.reshape(T, nh * d).contiguous(), 0, nh * d, packed, 0)
            ops.copy_columns(kh.reshape(T, nkv * d).contiguous(), 0, nkv * d, packed, nh * d)
            ops.copy_columns(qkv, (nh + nkv) * d, nkv * d, packed, (nh + nkv) * d)
            q = ops.qk_norm_rope_kv_write(packed, step.positions, slots, None, None,
                                          None, cache.kv, nh, nkv, d, 0, False, self.eps,
                                          write_kv=cache.writes)
        mfma = self.mfma and cache.kv.shape[3] % 4 == 0
        if mfma and step.n_tokens > step.n_seqs:
            # prompt portions in the step: both products on the matrix cores
            items = step.attention_items(self.mfma_rows_per_item)
            # a portion far into a long request yields few work items: cut its context
            keys, nsplit = plan_split(items[3], nkv, step.max_keys, target=BUSY_WORKGROUPS)
            # tiles of 128 keys spread a tile's fixed work over twice the scores (measured
            # faster from 512 tokens to 32,768); head size 128 keeps tiles of 64 (LDS)
            o = ops.paged_attention_mfma(q, cache.kv, step.block_tables[cache.group],
                                         step.positions, *items, self.scale, self.window,
                                         keys, nsplit, tile_keys=128 if d == 64 else 64)
        elif mfma:
            # single tokens only: the matrix-core kernel whose waves split the keys
            # (every request brings one token: row i is request i, no work-item arrays)
            item_seq = item_row0 = item_count = None
            n_items = step.n_seqs
            keys, nsplit = plan_split(n_items, nkv, step.max_keys)
            o = ops.paged_attention_decode_mfma(q, cache.kv, step.block_tables[cache.group],
                                                step.positions, item_seq, item_row0, item_count,
                                                n_items, self.scale, self.window, keys, nsplit)
        else:
            item_seq, item_row0, item_count, n_items = step.attention_items(self.rows_per_item)
            keys, nsplit = plan_split(n_items, nkv, step.max_keys)
            o = ops.paged_attention(q, cache.kv, step.block_tables[cache.group], step.positions,
                                    item_seq, item_row0, item_count, n_items, self.scale,
                                    self.window, keys, nsplit)
        if getattr(step, "taps", None) is not None:
            self._leave_taps(step, cache, q, o)
        return ops.linear(o.view(T, nh * d), self.w_out, self.b_out, partial_ok=True,
                          accumulate=stream, tune=self.runtime.tune)

    def _leave_taps(self, step, cache, q: torch.Tensor, o: torch.Tensor) -> None:
        """Diagnostics: the queries, the keys and values of the step's tokens as they lie in
        the cache now (read back through the tokens' places), and the attention's output."""
        step.taps["q"] = q.clone()
        step.taps["o"] = o.clone()
        if not cache.writes:
            return
        page_size = cache.kv.shape[3]
        place = step.slot_mapping[cache.group].long()
        page, offset = place // page_size, place % page_size
        step.taps["k"] = cache.kv[page, 0, :, offset, :]
        values = cache.kv[:, 1].reshape(cache.kv.shape[0], self.num_kv_heads, self.head_dim, page_size)
        step.taps["v"] = values[page, :, :, offset]


register_mixer(GroupedQueryAttention.kind, GroupedQueryAttention)
