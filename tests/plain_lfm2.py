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
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

DT = torch.float64


# ------------------------------------------------ where a bfloat16 run rounds
def bf(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 (nearest even) and widen again."""
    return x.to(torch.bfloat16).to(x.dtype)


@dataclass
class Rounding:
    """Where a bfloat16 run of the model stores bfloat16 between its 32-bit sums, so that
    the plain implementation can round at the same places (sums, norms, softmax, the
    residual stream and the logits stay wide).  Always rounded: a norm's output, the
    opening projections' outputs (q|k|v, B|C|x), q and k after the rotation, the
    attention's output, the convolution's gated output, the SwiGLU's output.  What depends
    on how a token was run is given per position (one boolean per row, ``True`` for the
    form that a step of few tokens takes):

      late_norm[key]   the product applies the row's scale itself:
                       y = scale * (bf(x * w) @ W^T)  instead of  bf(x * scale * w) @ W^T;
                       keys (layer, "mixer"), (layer, "feed_forward") and "head"
      wide_gate        the SwiGLU gate is applied to the unrounded gate and up products
      wide_close[key]  the closing product (out_proj, w2) is added to the stream as the
                       32-bit sum it is, not rounded first; keys (layer, "mixer"),
                       (layer, "feed_forward")

    ``probabilities``: the attention rounds its probabilities for the second product
    (the sum they are divided by stays unrounded).  A missing key means ``False``
    everywhere."""

    late_norm: Dict[object, torch.Tensor] = field(default_factory=dict)
    wide_gate: Optional[torch.Tensor] = None
    wide_close: Dict[object, torch.Tensor] = field(default_factory=dict)
    probabilities: bool = True

    @staticmethod
    def _rows(mask: Optional[torch.Tensor], n: int) -> torch.Tensor:
        return torch.zeros(n, dtype=torch.bool) if mask is None else mask.to(torch.bool)


def by_row(mask: torch.Tensor, when_true, when_false) -> torch.Tensor:
    """Rows of ``when_true()`` where ``mask`` holds and of ``when_false()`` elsewhere; each
    is called with the row indices it has to produce and only if there are any."""
    yes, no = mask.nonzero().flatten(), (~mask).nonzero().flatten()
    if yes.numel() == 0:
        return when_false(no)
    if no.numel() == 0:
        return when_true(yes)
    a, b = when_true(yes), when_false(no)
    out = torch.empty((mask.numel(),) + tuple(a.shape[1:]), dtype=a.dtype)
    out[yes], out[no] = a, b
    return out


def normed_product(x: torch.Tensor, norm_w: torch.Tensor, eps: float, W: torch.Tensor,
                   bias: Optional[torch.Tensor], rounding: Optional[Rounding],
                   late: Optional[torch.Tensor]) -> torch.Tensor:
    """``rms_norm(x) @ W^T + bias`` (norm.zig:6-33, then the projection), unrounded
    result; with ``rounding`` the operand is rounded where a bfloat16 run rounds it."""
    def add_bias(y):
        return y if bias is None else y + bias
    if rounding is None:
        return add_bias(rms_norm(x, norm_w, eps) @ W.T)

    def early(rows):
        return add_bias(bf(rms_norm(x[rows], norm_w, eps)) @ W.T)

    def late_form(rows):
        xr = x[rows]
        scale = 1.0 / torch.sqrt((xr * xr).sum(dim=-1, keepdim=True) / xr.shape[-1] + eps)
        return add_bias((bf(xr * norm_w) @ W.T) * scale)

    return by_row(Rounding._rows(late, x.shape[0]), late_form, early)


# ------------------------------------------------------------------ the parts
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """norm.zig:6-33: ms = sum(x^2)/n; scale = 1/sqrt(ms + eps); out = x*scale*w."""
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(ms + eps)) * w


def rope_inv_freq(rotary_dim: int, theta: float, dtype=DT) -> torch.Tensor:
    """rope.zig:29-32: freq_i = 1 / base^(2i / dim), i < dim/2."""
    i = torch.arange(0, rotary_dim // 2, dtype=DT)
    return (1.0 / torch.pow(torch.tensor(theta, dtype=DT), 2.0 * i / rotary_dim)).to(dtype)


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
                     scale: Optional[float] = None, round_probabilities: bool = False) -> torch.Tensor:
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
        if round_probabilities:
            # A bfloat16 run on the matrix cores rounds the unnormalised probabilities for
            # the second product and divides by the sum of the rounded values (the weights
            # that reach the values then add up to one).  It takes them
            # relative to the row's maximum rounded up to a whole number on the base-2
            # scale, p = 2^(s log2(e) - ceil(max)): the same softmax (the common factor
            # cancels), and the one form in which the rounded values do not depend on the
            # order in which the keys are visited.
            t = s * math.log2(math.e)
            p = torch.exp2(t - torch.ceil(t.max(dim=-1, keepdim=True).values))
            p = bf(p)
            out[:, h, :] = (p @ v[:, g, :]) / p.sum(dim=-1, keepdim=True)
        else:
            p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
            out[:, h, :] = (p / p.sum(dim=-1, keepdim=True)) @ v[:, g, :]
    return out


def attention_mixer(x: torch.Tensor, w: Dict[str, torch.Tensor], positions: torch.Tensor,
                    num_heads: int, num_kv_heads: int, head_dim: int, eps: float, theta: float,
                    window: int = 0) -> torch.Tensor:
    """hybrid_attn.zig:286-640: projections (no bias), per-head RMSNorm of q and k
    (371-382, before the rotation, not on v), RoPE, causal softmax attention,
    output projection."""
    qkv = x @ torch.cat([w["q_proj"], w["k_proj"], w["v_proj"]]).T
    return attention_core(qkv, w, positions, num_heads, num_kv_heads, head_dim, eps, theta,
                          window) @ w["out_proj"].T


def attention_inputs(qkv: torch.Tensor, w: Dict[str, torch.Tensor], positions: torch.Tensor,
                     num_heads: int, num_kv_heads: int, head_dim: int, eps: float, theta: float,
                     rounding: Optional[Rounding] = None):
    """The projected q|k|v rows as heads: q and k normalised per head and rotated
    (hybrid_attn.zig:362-396), v as it is.  With ``rounding`` q and k are rounded after the
    rotation (they are stored so)."""
    T = qkv.shape[0]
    nq, nk = num_heads * head_dim, num_kv_heads * head_dim
    q = qkv[:, :nq].reshape(T, num_heads, head_dim)
    k = qkv[:, nq:nq + nk].reshape(T, num_kv_heads, head_dim)
    v = qkv[:, nq + nk:].reshape(T, num_kv_heads, head_dim)
    q = apply_rope(rms_norm(q, w["q_norm"], eps), positions, theta)
    k = apply_rope(rms_norm(k, w["k_norm"], eps), positions, theta)
    if rounding is not None:
        q, k = bf(q), bf(k)
    return q, k, v


def attention_core(qkv: torch.Tensor, w: Dict[str, torch.Tensor], positions: torch.Tensor,
                   num_heads: int, num_kv_heads: int, head_dim: int, eps: float, theta: float,
                   window: int = 0, rounding: Optional[Rounding] = None) -> torch.Tensor:
    """From the projected q|k|v rows to the attention's output ``[T, heads * head_dim]``
    (hybrid_attn.zig:362-608).  With ``rounding``: the probabilities are rounded if the
    run rounds them, and the output."""
    q, k, v = attention_inputs(qkv, w, positions, num_heads, num_kv_heads, head_dim, eps, theta,
                               rounding)
    return attention_output(q, k, v, positions, window, rounding)


def attention_output(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
                     window: int = 0, rounding: Optional[Rounding] = None) -> torch.Tensor:
    o = causal_attention(q, k, v, positions, window,
                         round_probabilities=rounding is not None and rounding.probabilities)
    o = o.reshape(q.shape[0], q.shape[1] * q.shape[2])
    return bf(o) if rounding is not None else o


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
    y = short_conv_core(z, w) @ w["out_proj"].T
    if "out_proj_bias" in w:
        y = y + w["out_proj_bias"]
    return y


def short_conv_core(z: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    """From the projected B|C|x rows to the gated convolution's output ``[T, H]``."""
    H = z.shape[1] // 3
    B, C, xx = z[:, :H], z[:, H:2 * H], z[:, 2 * H:]
    return C * causal_depthwise_conv(B * xx, w["conv"], w.get("conv_bias"))


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

    def attention_qkv(self, i: int, x: torch.Tensor, positions: torch.Tensor,
                      rounding: Optional[Rounding] = None):
        """Layer ``i``'s queries, keys and values ``[T, heads, head_dim]`` from the stream:
        what the attention reads (the queries) and what goes into the cache."""
        lw = self.layer_weights(i)
        w_qkv = torch.cat([lw["q_proj"], lw["k_proj"], lw["v_proj"]])
        late = rounding.late_norm.get((i, "mixer")) if rounding is not None else None
        qkv = normed_product(x, self.w[f"model.layers.{i}.operator_norm.weight"], self.eps, w_qkv,
                             None, rounding, late)
        if rounding is not None:
            qkv = bf(qkv)
        return attention_inputs(qkv, lw, positions, self.nh, self.nkv, self.d, self.eps,
                                self.theta, rounding)

    def layer(self, i: int, x: torch.Tensor, positions: torch.Tensor,
              rounding: Optional[Rounding] = None,
              attention_output_given: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decoder block on the whole sequence's stream ``x [T, H]``
        (hybrid_layer.zig:366-492): h = x + mixer(norm1(x)); y = h + ffn(norm2(h)).
        With ``rounding`` the same formulas, rounded to bfloat16 where such a run stores
        bfloat16 (see ``Rounding``).  ``attention_output_given`` ``[T, heads * head_dim]``
        stands in for the attention's output (tests that look at the rest of the block
        alone)."""
        w = self.w
        p = f"model.layers.{i}."
        lw = self.layer_weights(i)
        if rounding is None:
            n1 = rms_norm(x, w[p + "operator_norm.weight"], self.eps)
            if self.kinds[i] == "attention" and attention_output_given is not None:
                m = attention_output_given.to(x.dtype) @ lw["out_proj"].T
            elif self.kinds[i] == "attention":
                m = attention_mixer(n1, lw, positions, self.nh, self.nkv, self.d, self.eps,
                                    self.theta)
            else:
                m = short_conv_mixer(n1, lw)
            h = x + m
            n2 = rms_norm(h, w[p + "ffn_norm.weight"], self.eps)
            return h + swiglu_ffn(n2, w[p + "feed_forward.w1.weight"],
                                  w[p + "feed_forward.w3.weight"], w[p + "feed_forward.w2.weight"])
        r = rounding
        T = x.shape[0]

        def closing(y, key):
            wide = Rounding._rows(r.wide_close.get(key), T)
            return torch.where(wide[:, None], y, bf(y))

        late = r.late_norm.get((i, "mixer"))
        if self.kinds[i] == "attention":
            if attention_output_given is not None:
                o = attention_output_given.to(x.dtype)
            else:
                q, k, v = self.attention_qkv(i, x, positions, r)
                o = attention_output(q, k, v, positions, 0, r)
            m = o @ lw["out_proj"].T
        else:
            z = bf(normed_product(x, w[p + "operator_norm.weight"], self.eps, lw["in_proj"],
                                  lw.get("in_proj_bias"), r, late))
            m = bf(short_conv_core(z, lw)) @ lw["out_proj"].T
            if "out_proj_bias" in lw:
                m = m + lw["out_proj_bias"]
        h = x + closing(m, (i, "mixer"))
        w_gu = torch.cat([w[p + "feed_forward.w1.weight"], w[p + "feed_forward.w3.weight"]])
        gu = normed_product(h, w[p + "ffn_norm.weight"], self.eps, w_gu, None, r,
                            r.late_norm.get((i, "feed_forward")))
        gu = torch.where(Rounding._rows(r.wide_gate, T)[:, None], gu, bf(gu))
        inter = gu.shape[1] // 2
        g, u = gu[:, :inter], gu[:, inter:]
        a = bf(g * (1.0 / (1.0 + torch.exp(-g))) * u)
        return h + closing(a @ w[p + "feed_forward.w2.weight"].T, (i, "feed_forward"))

    def embed(self, tokens: Sequence[int]) -> torch.Tensor:
        return embedding(tokens, self.w["model.embed_tokens.weight"])

    def hidden_states(self, tokens: Sequence[int], position_offset: int = 0,
                      upto_layer: Optional[int] = None,
                      rounding: Optional[Rounding] = None) -> torch.Tensor:
        x = self.embed(tokens)
        positions = torch.arange(len(tokens)) + position_offset
        n_layers = len(self.kinds) if upto_layer is None else upto_layer
        for i in range(n_layers):
            x = self.layer(i, x, positions, rounding)
        return x

    def head(self, x: torch.Tensor, rounding: Optional[Rounding] = None,
             late: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Final RMSNorm, then the output projection (tied: the embedding table;
        gguf_model.zig:47-54, main.zig:870-877) of the rows ``x`` of the stream."""
        table = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return normed_product(x, self.w["model.embedding_norm.weight"], self.eps, table, None,
                              rounding, late)

    def logits(self, tokens: Sequence[int], rows: Optional[Sequence[int]] = None,
               rounding: Optional[Rounding] = None) -> torch.Tensor:
        """Logits of all positions, or of ``rows``."""
        x = self.hidden_states(tokens, rounding=rounding)
        late = rounding.late_norm.get("head") if rounding is not None else None
        if rows is not None:
            idx = torch.as_tensor(list(rows), dtype=torch.long)
            x = x[idx]
            late = late[idx] if late is not None else None
        return self.head(x, rounding, late)

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
