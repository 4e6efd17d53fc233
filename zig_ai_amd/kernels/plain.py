"""The plain C++ statements of the kernels (``csrc/plain.cpp``) behind functions that
take and return float32 tensors on the CPU, with the operands of the kernels'
own wrappers in ``ops``.  For checking kernels and layouts; the engine does not
import this module.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p
from typing import Optional, Tuple

import torch

from . import build

_SIGNATURES = {
    "za_plain_add_rmsnorm": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_float],
    "za_plain_embed": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int],
    "za_plain_linear": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int],
    "za_plain_swiglu": [c_void_p, c_void_p, c_int, c_int],
    "za_plain_qk_norm_rope_kv_write": [c_void_p] * 8 + [c_int] * 6 + [c_float, c_int, c_int],
    "za_plain_paged_attention": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_float, c_int],
    "za_plain_short_conv": [c_void_p] * 7 + [c_int, c_int, c_int],
    "za_plain_argmax": [c_void_p, c_int, c_int, c_void_p],
    "za_plain_repetition_penalty": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int],
    "za_plain_sample_weights": [c_void_p, c_int, c_float, c_int, c_float, c_void_p, c_void_p],
    "za_plain_sample": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
}

_lib: Optional[ctypes.CDLL] = None


class PlainError(ValueError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        loaded = build.load("plain")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(loaded, name)
            fn.restype = c_int
            fn.argtypes = argtypes
        _lib = loaded
    return _lib


def _f32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.device.type != "cpu" or t.dtype != torch.float32 or not t.is_contiguous():
        raise PlainError(f"{name} must be a contiguous float32 tensor on the CPU")
    return t


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.device.type != "cpu" or t.dtype != torch.int32 or not t.is_contiguous():
        raise PlainError(f"{name} must be a contiguous int32 tensor on the CPU")
    return t


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _call(name: str, *args) -> None:
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise PlainError(f"{name} refused its arguments")


def add_rmsnorm(residual: Optional[torch.Tensor], delta: Optional[torch.Tensor],
                weight: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(residual + sum of delta's terms, its RMSNorm)``; ``delta`` is ``[T, H]`` or a
    stack ``[P, T, H]``; with ``residual=None`` the sum is ``delta`` alone."""
    ref = residual if residual is not None else delta
    T, H = ref.shape[-2], ref.shape[-1]
    P = 0
    if delta is not None:
        _f32(delta, "delta")
        P = delta.shape[0] if delta.dim() == 3 else 1
    if residual is not None:
        new_res = _f32(residual, "residual").clone()
    else:
        new_res = torch.zeros((T, H), dtype=torch.float32)
    out = torch.empty((T, H), dtype=torch.float32)
    _call("za_plain_add_rmsnorm", _p(new_res), _p(delta), P, _p(_f32(weight, "weight")), _p(out),
          T, H, float(eps))
    return new_res, out


def embed(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    out = torch.empty((tokens.numel(), table.shape[1]), dtype=torch.float32)
    _call("za_plain_embed", _p(_i32(tokens, "tokens")), _p(_f32(table, "table")), _p(out),
          tokens.numel(), table.shape[1], table.shape[0])
    return out


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    M, K = x.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise PlainError("weight must be [N, K]")
    y = torch.empty((M, N), dtype=torch.float32)
    _call("za_plain_linear", _p(_f32(x, "x")), _p(_f32(weight, "weight")),
          _p(None if bias is None else _f32(bias, "bias")), _p(y), M, N, K)
    return y


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    T, two_i = gate_up.shape
    out = torch.empty((T, two_i // 2), dtype=torch.float32)
    _call("za_plain_swiglu", _p(_f32(gate_up, "gate_up")), _p(out), T, two_i // 2)
    return out


def qk_norm_rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                          q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor],
                          inv_freq: Optional[torch.Tensor], kv_cache: Optional[torch.Tensor],
                          num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int,
                          adjacent_pairs: bool, eps: float, write_kv: bool = True) -> torch.Tensor:
    """Queries ``[T, heads, head_dim]``; ``kv_cache [pages, 2, kv_heads, page_size,
    head_dim]`` is written in place (a page's value half holds ``[head_dim][offset]``)."""
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise PlainError("qkv has the wrong width")
    page_size = kv_cache.shape[3] if write_kv else 0
    q_out = torch.empty((T, num_heads, head_dim), dtype=torch.float32)
    _call("za_plain_qk_norm_rope_kv_write", _p(_f32(qkv, "qkv")), _p(_i32(positions, "positions")),
          _p(_i32(slots, "slots")) if write_kv else None,
          _p(None if q_norm_w is None else _f32(q_norm_w, "q_norm_w")),
          _p(None if k_norm_w is None else _f32(k_norm_w, "k_norm_w")),
          _p(_f32(inv_freq, "inv_freq")) if rotary_dim else None, _p(q_out),
          _p(_f32(kv_cache, "kv_cache")) if write_kv else None, T, num_heads, num_kv_heads,
          head_dim, rotary_dim, 1 if adjacent_pairs else 0, float(eps), page_size,
          1 if write_kv else 0)
    return q_out


def paged_attention(q: torch.Tensor, kv_cache: torch.Tensor, block_table: torch.Tensor,
                    positions: torch.Tensor, token_seq: torch.Tensor, scale: float,
                    window: int = 0) -> torch.Tensor:
    """Token ``t`` (request ``token_seq[t]``, position ``positions[t]``) over its
    request's keys in the cache."""
    T, nh, d = q.shape
    nkv, page_size = kv_cache.shape[2], kv_cache.shape[3]
    out = torch.empty_like(q)
    _call("za_plain_paged_attention", _p(_f32(q, "q")), _p(out), _p(_f32(kv_cache, "kv_cache")),
          _p(_i32(block_table, "block_table")), block_table.shape[1],
          _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")), T, nh, nkv, d,
          page_size, float(scale), int(window))
    return out


def short_conv(z: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               state: torch.Tensor, seq_start: torch.Tensor, slot_id: torch.Tensor) -> torch.Tensor:
    """``weight [width, L]`` as a checkpoint holds it; ``state [slots, width, L]`` is
    updated in place; ``seq_start`` has one entry more than ``slot_id``."""
    width, L = weight.shape
    T = z.shape[0]
    if z.shape[1] != 3 * width or tuple(state.shape[1:]) != (width, L):
        raise PlainError("z or state has the wrong shape")
    if seq_start.numel() != slot_id.numel() + 1 or int(seq_start[-1]) != T:
        raise PlainError("seq_start must list the start of every request and the end of the last")
    y = torch.empty((T, width), dtype=torch.float32)
    _call("za_plain_short_conv", _p(_f32(z, "z")), _p(_f32(weight, "weight")),
          _p(None if bias is None else _f32(bias, "bias")), _p(_f32(state, "state")),
          _p(_i32(seq_start, "seq_start")), _p(_i32(slot_id, "slot_id")), _p(y), slot_id.numel(),
          width, L)
    return y


def argmax(logits: torch.Tensor) -> torch.Tensor:
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32)
    _call("za_plain_argmax", _p(_f32(logits, "logits")), R, V, _p(out))
    return out


def repetition_penalty_(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor,
                        factors: torch.Tensor) -> None:
    _call("za_plain_repetition_penalty", _p(_f32(logits, "logits")), logits.shape[1],
          _p(_i32(rows, "rows")), _p(_i32(tokens, "tokens")), _p(_f32(factors, "factors")),
          rows.numel())


def sample_weights(row: torch.Tensor, temperature: float, top_k: int,
                   top_p: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(weight [vocab] float64, keep [vocab] bool)`` of one row."""
    V = row.numel()
    weight = torch.empty((V,), dtype=torch.float64)
    keep = torch.empty((V,), dtype=torch.uint8)
    _call("za_plain_sample_weights", _p(_f32(row, "row")), V, float(temperature), int(top_k),
          float(top_p), _p(weight), _p(keep))
    return weight, keep.bool()


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32)
    _call("za_plain_sample", _p(_f32(logits, "logits")), R, V, _p(_f32(temperature, "temperature")),
          _p(_i32(top_k, "top_k")), _p(_f32(top_p, "top_p")), _p(_f32(uniform, "uniform")), _p(out))
    return out
