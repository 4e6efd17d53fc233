"""A plain, slow LFM2: whole sequences, no cache, no batching, one function per
part, on the CPU in float64 (or any dtype given).  It shares no code with the
engine: it reads config.json and the safetensors file itself (through the
safetensors package) and knows the checkpoint names by itself.

Each function cites the reference lines its formula was read from
(/root/reference, read, never run).  Where the reference's LFM2 path departs
from the model's definition (its ShortConv applies the convolution before the
projection, with SiLU and a different gate, short_conv.zig:174-277), the
definition stated for this engine governs: in_proj -> (B, C, x); B*x; causal
depth-wise convolution of conv_L_cache taps; *C; out_proj.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

DT = torch.float64


# ------------------------------------------------------------------ the parts
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """norm.zig:6-33: ms = sum(x^2)/n; scale = 1/sqrt(ms + eps); out = x*scale*w."""
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(ms + eps)) * w


def rope_inv_freq(rotary_dim: int, theta: float, dtype=DT) -> torch.Tensor:
    """rope.zig:29-32: freq_i = 1 / base^(2i / dim), i < dim/2."""
    i = torch.arange(0, rotary_dim // 2, dtype=dtype)
    return 1.0 / torch.pow(torch.tensor(theta, dtype=dtype), 2.0 * i / rotary_dim)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, theta: float,
               rotary_dim: Optional[int] = None, pairing: str = "half") -> torch.Tensor:
    """x: [T, heads, d].  rope.zig:40-56: angle = pos * freq_i;
    (a, b) -> (a cos - b sin, a sin + b cos).  Pairs are (i, i + rot/2) for "half"
    (the reference's device kernel, layer_kernels.cu:353-365) or (2i, 2i+1) for
    "adjacent" (rope.zig:46-53).  Elements past rotary_dim are untouched."""
    d = x.shape[-1]
    rot = d if rotary_dim is None else rotary_dim
    inv = rope_inv_freq(rot, theta, x.dtype)
    ang = positions.to(x.dtype)[:, None] * inv[None, :]          # [T, rot/2]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if pairing == "half":
        a, b = x[..., : rot // 2], x[..., rot // 2: rot]
        out[..., : rot // 2] = a * cos - b * sin
        out[..., rot // 2: rot] = a * sin + b * cos
    elif pairing == "adjacent":
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        out[..., 0:rot:2] = a * cos - b * sin
        out[..., 1:rot:2] = a * sin + b * cos
    else:
        raise ValueError(pairing)
    return out


def kv_head_of(h: int, num_heads: int, num_kv_heads: int) -> int:
    """gqa.zig:12-36 / hybrid_attn.zig:553: kv = h / (nh / nkv)."""
    return h // (num_heads // num_kv_heads)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     positions: Optional[torch.Tensor] = None, window: int = 0,
                     scale: Optional[float] = None) -> torch.Tensor:
    """q: [T, nh, d]; k, v: [T, nkv, d] (the whole sequence).  hybrid_attn.zig:571-608:
    s = q.k / sqrt(d), keys after the query masked, two-pass softmax, weighted
    sum of values.  ``window`` > 0 also masks keys at distance >= window."""
    T, nh, d = q.shape
    nkv = k.shape[1]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    pos = torch.arange(T) if positions is None else positions
    out = torch.zeros_like(q)
    for h in range(nh):
        g = kv_head_of(h, nh, nkv)
        s = (q[:, h, :] @ k[:, g, :].T) * scale                  # [T, T]
        dist = pos[:, None] - pos[None, :]
        mask = dist < 0
        if window > 0:
            mask = mask | (dist >= window)
        s = s.masked_fill(mask, float("-inf"))
        p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def attention_mixer(x: torch.Tensor, w: Dict[str, torch.Tensor], positions: torch.Tensor,
                    num_heads: int, num_kv_heads: int, head_dim: int, eps: float, theta: float,
                    window: int = 0) -> torch.Tensor:
    """hybrid_attn.zig:286-640: projections (no bias), per-head RMSNorm of q and k
    (371-382, before the rotation, not on v), RoPE, causal softmax attention,
    output projection."""
    T = x.shape[0]
    q = (x @ w["q_proj"].T).view(T, num_heads, head_dim)
    k = (x @ w["k_proj"].T).view(T, num_kv_heads, head_dim)
    v = (x @ w["v_proj"].T).view(T, num_kv_heads, head_dim)
    q = rms_norm(q, w["q_norm"], eps)
    k = rms_norm(k, w["k_norm"], eps)
    q = apply_rope(q, positions, theta)
    k = apply_rope(k, positions, theta)
    o = causal_attention(q, k, v, positions, window)
    return o.reshape(T, num_heads * head_dim) @ w["out_proj"].T


def causal_depthwise_conv(u: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """u: [T, H]; w: [H, L].  c[t] = bias + sum_j w[:, j] * u[t - (L-1) + j], zeros
    before the sequence (the mechanics of layer_kernels.cu:192-222 with a zero
    state, taps over the L most recent inputs)."""
    T, H = u.shape
    L = w.shape[1]
    padded = torch.cat([torch.zeros(L - 1, H, dtype=u.dtype), u], dim=0)
    c = torch.zeros_like(u)
    for j in range(L):
        c = c + padded[j: j + T, :] * w[:, j][None, :]
    if bias is not None:
        c = c + bias[None, :]
    return c


def short_conv_mixer(x: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    """in_proj -> (B, C, x) in that order; u = B*x; causal depth-wise conv; y = C*c;
    out_proj.  Biases on all three when present."""
    z = x @ w["in_proj"].T
    if "in_proj_bias" in w:
        z = z + w["in_proj_bias"]
    H = x.shape[1]
    B, C, xx = z[:, :H], z[:, H:2 * H], z[:, 2 * H:]
    c = causal_depthwise_conv(B * xx, w["conv"], w.get("conv_bias"))
    y = (C * c) @ w["out_proj"].T
    if "out_proj_bias" in w:
        y = y + w["out_proj_bias"]
    return y


def swiglu_ffn(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
               w_down: torch.Tensor) -> torch.Tensor:
    """ffn.zig:19-33: (silu(x Wg^T) * (x Wu^T)) Wd^T, silu(g) = g * sigmoid(g)."""
    g = x @ w_gate.T
    u = x @ w_up.T
    return (g * (1.0 / (1.0 + torch.exp(-g))) * u) @ w_down.T


def embedding(tokens: Sequence[int], table: torch.Tensor) -> torch.Tensor:
    """embedding.zig:21-30: row gather (the reference clamps ids, here they must be
    in range)."""
    idx = torch.as_tensor(list(tokens), dtype=torch.long)
    assert int(idx.min()) >= 0 and int(idx.max()) < table.shape[0]
    return table[idx]


def ffn_width(cfg: dict) -> int:
    """Two thirds, optional multiplier, rounded up to multiple_of when
    block_auto_adjust_ff_dim is on (12288 -> 8192 at 256; 384 -> 256 at 128)."""
    width = cfg.get("block_ff_dim", cfg.get("intermediate_size"))
    if cfg.get("block_auto_adjust_ff_dim", True):
        width = int(2 * width / 3)
        if cfg.get("block_ffn_dim_multiplier") is not None:
            width = int(cfg["block_ffn_dim_multiplier"] * width)
        m = cfg["block_multiple_of"]
        width = m * ((width + m - 1) // m)
    return width


# -------------------------------------------------------------- the whole model
class PlainLfm2:
    def __init__(self, model_dir: str, dtype=DT):
        from safetensors.torch import load_file
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        raw = load_file(os.path.join(model_dir, "model.safetensors"))
        self.w = {k: v.to(dtype) for k, v in raw.items()}
        self.dtype = dtype
        c = self.cfg
        self.H = c["hidden_size"]
        self.nh = c["num_attention_heads"]
        self.nkv = c.get("num_key_value_heads", self.nh)
        self.d = c.get("head_dim", self.H // self.nh)
        self.eps = c["norm_eps"]
        self.theta = c["rope_theta"]
        self.kinds = ["attention" if t in ("full_attention", "attention") else "conv"
                      for t in c["layer_types"]]
        self.tied = c.get("tie_embedding", c.get("tie_word_embeddings", True))

    def layer_weights(self, i: int) -> Dict[str, torch.Tensor]:
        p = f"model.layers.{i}."
        w = self.w
        if self.kinds[i] == "attention":
            return {"q_proj": w[p + "self_attn.q_proj.weight"], "k_proj": w[p + "self_attn.k_proj.weight"],
                    "v_proj": w[p + "self_attn.v_proj.weight"],
                    "out_proj": w[p + "self_attn.out_proj.weight"],
                    "q_norm": w[p + "self_attn.q_layernorm.weight"],
                    "k_norm": w[p + "self_attn.k_layernorm.weight"]}
        out = {"in_proj": w[p + "conv.in_proj.weight"],
               "conv": w[p + "conv.conv.weight"].reshape(self.H, -1),
               "out_proj": w[p + "conv.out_proj.weight"]}
        for local, name in (("in_proj_bias", "conv.in_proj.bias"), ("conv_bias", "conv.conv.bias"),
                            ("out_proj_bias", "conv.out_proj.bias")):
            if p + name in w:
                out[local] = w[p + name]
        return out

    def hidden_states(self, tokens: Sequence[int], position_offset: int = 0,
                      upto_layer: Optional[int] = None) -> torch.Tensor:
        """hybrid_layer.zig:366-492: h = x + mixer(norm1(x)); y = h + ffn(norm2(h))."""
        w = self.w
        x = embedding(tokens, w["model.embed_tokens.weight"])
        positions = torch.arange(len(tokens)) + position_offset
        n_layers = len(self.kinds) if upto_layer is None else upto_layer
        for i in range(n_layers):
            p = f"model.layers.{i}."
            n1 = rms_norm(x, w[p + "operator_norm.weight"], self.eps)
            lw = self.layer_weights(i)
            if self.kinds[i] == "attention":
                m = attention_mixer(n1, lw, positions, self.nh, self.nkv, self.d, self.eps,
                                    self.theta)
            else:
                m = short_conv_mixer(n1, lw)
            h = x + m
            n2 = rms_norm(h, w[p + "ffn_norm.weight"], self.eps)
            f = swiglu_ffn(n2, w[p + "feed_forward.w1.weight"], w[p + "feed_forward.w3.weight"],
                           w[p + "feed_forward.w2.weight"])
            x = h + f
        return x

    def logits(self, tokens: Sequence[int]) -> torch.Tensor:
        """Final RMSNorm, then the output projection (tied: the embedding table;
        gguf_model.zig:47-54, main.zig:870-877)."""
        x = self.hidden_states(tokens)
        n = rms_norm(x, self.w["model.embedding_norm.weight"], self.eps)
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return n @ head.T

    def greedy(self, prompt: Sequence[int], n_new: int) -> List[int]:
        toks = list(prompt)
        out = []
        for _ in range(n_new):
            nxt = argmax_first(self.logits(toks)[-1])
            out.append(nxt)
            toks.append(nxt)
        return out


# ------------------------------------------------------------------- sampling
def argmax_first(logits: torch.Tensor) -> int:
    """pipeline.zig:155-181: the first index of the maximum."""
    best, idx = -math.inf, 0
    for i, v in enumerate(logits.tolist()):
        if v > best:
            best, idx = v, i
    return idx


def apply_repetition_penalty(logits: torch.Tensor, history: Sequence[int], penalty: float) -> torch.Tensor:
    """pipeline.zig:61-68: once per occurrence in the history, positive logits are
    divided by the penalty and negative ones multiplied."""
    out = logits.clone()
    for tok in history:
        if 0 <= tok < out.numel():
            if out[tok] > 0:
                out[tok] = out[tok] / penalty
            elif out[tok] < 0:
                out[tok] = out[tok] * penalty
    return out


def kept_after_top_k_top_p(scaled: torch.Tensor, top_k: int, top_p: float) -> torch.Tensor:
    """Boolean mask of the candidates.  pipeline.zig:80-99: top-k keeps values >=
    the k-th largest; 102-142: top-p keeps the shortest descending prefix whose
    probability reaches p (ties with its last value kept as well)."""
    V = scaled.numel()
    keep = torch.ones(V, dtype=torch.bool)
    if 0 < top_k < V:
        kth = torch.sort(scaled, descending=True).values[top_k - 1]
        keep = scaled >= kth
    if top_p < 1.0:
        vals = scaled.masked_fill(~keep, float("-inf"))
        order = torch.argsort(vals, descending=True)
        probs = torch.softmax(vals[order], dim=0)
        cum = torch.cumsum(probs, dim=0)
        cutoff = int((cum >= top_p).nonzero()[0]) + 1 if bool((cum >= top_p).any()) else V
        last = vals[order][cutoff - 1]
        keep = keep & (vals >= last)
    return keep


def sample_token(logits: torch.Tensor, temperature: float, u: float, top_k: int = 0,
                 top_p: float = 1.0) -> int:
    """pipeline.zig:39-52: greedy when temperature <= 0; else with v = logit / T and
    m = max v, the first index i (in index order, over the kept candidates) whose
    cumulative sum of exp(v - m) reaches u * total; the last candidate if none."""
    if temperature <= 0:
        return argmax_first(logits)
    v = logits.to(DT) / temperature
    keep = kept_after_top_k_top_p(v, top_k, top_p)
    e = torch.where(keep, torch.exp(v - v[keep].max()), torch.zeros_like(v))
    total = float(e.sum())
    target = u * total
    acc = 0.0
    last = 0
    for i, x in enumerate(e.tolist()):
        if x > 0:
            acc += x
            last = i
            if target <= acc:
                return i
    return last
