"""Typed configuration of the LFM2 ShortConv/attention hybrid, read from the
keys of its config.json.

The reference derives the same facts from GGUF metadata
(/root/reference/src/loader/model_config.zig:46-131, lfm2 branch 97-128: a
per-layer attention flag array and ``shortconv_l_cache``); here they come from
config.json: ``layer_types`` (or the older ``full_attn_idxs``), ``conv_L_cache``,
``conv_bias``, ``block_ff_dim`` with ``block_auto_adjust_ff_dim`` /
``block_multiple_of`` / ``block_ffn_dim_multiplier``, and the usual sizes.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .fields import (has_any, read_bool, read_float, read_int, read_int_list,
                     read_str_list)
from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

ATTENTION_NAMES = ("full_attention", "attention", "attn")
CONV_NAMES = ("conv", "short_conv", "shortconv")


def feed_forward_width(block_ff_dim: int, auto_adjust: bool, multiple_of: Optional[int],
                       multiplier: Optional[float]) -> int:
    """Width of the SwiGLU hidden layer.

    With auto-adjust the configured width is first cut to two thirds (the
    gate/up pair replaces one matrix of a plain MLP), optionally scaled, and
    rounded up to a multiple of ``multiple_of``: 12288 -> 8192, 6656 -> 4608,
    10752 -> 7168 at 256; 384 -> 256 at 128.
    """
    width = block_ff_dim
    if auto_adjust:
        if multiple_of is None:
            raise ConfigError("block_auto_adjust_ff_dim needs block_multiple_of")
        width = int(2 * width / 3)
        if multiplier is not None:
            width = int(multiplier * width)
        width = multiple_of * ((width + multiple_of - 1) // multiple_of)
    return width


def _with_nested_rope(data: Mapping[str, Any]) -> Mapping[str, Any]:
    """Some writers put the rotary base under ``rope_parameters`` / ``rope_scaling``."""
    if "rope_theta" in data and data["rope_theta"] is not None:
        return data
    for key in ("rope_parameters", "rope_scaling"):
        nested = data.get(key)
        if isinstance(nested, Mapping) and nested.get("rope_theta") is not None:
            return {**data, "rope_theta": nested["rope_theta"]}
    return data


@dataclass(frozen=True)
class Lfm2Config:
    architecture: str
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    vocab_size: int
    layer_types: Tuple[str, ...]          # "conv" | "attention", one per layer
    block_ff_dim: int
    auto_adjust_ff_dim: bool
    multiple_of: Optional[int]
    ffn_dim_multiplier: Optional[float]
    intermediate_size: int                # derived, after auto-adjust
    rope_theta: float
    norm_eps: float
    conv_L_cache: int
    conv_bias: bool
    tie_embedding: bool
    max_position_embeddings: int
    eos_token_id: Optional[int]

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "Lfm2Config":
        archs = data.get("architectures") or ["Lfm2ForCausalLM"]
        hidden = read_int(data, ["hidden_size"], minimum=1)
        n_layers = read_int(data, ["num_hidden_layers"], minimum=1)
        n_heads = read_int(data, ["num_attention_heads", "num_heads"], minimum=1)
        n_kv = read_int(data, ["num_key_value_heads"], default=n_heads, minimum=1)
        if has_any(data, ["head_dim"]):
            head_dim = read_int(data, ["head_dim"], minimum=1)
        else:
            if hidden % n_heads:
                raise ConfigError(
                    f"hidden_size {hidden} is not a multiple of num_attention_heads {n_heads} "
                    "and head_dim is not given")
            head_dim = hidden // n_heads
        if n_heads % n_kv:
            raise ConfigError(
                f"num_attention_heads {n_heads} is not a multiple of num_key_value_heads {n_kv}")
        vocab = read_int(data, ["vocab_size"], minimum=1)

        if has_any(data, ["layer_types"]):
            names = read_str_list(data, ["layer_types"])
            kinds = []
            for i, name in enumerate(names):
                if name in ATTENTION_NAMES:
                    kinds.append("attention")
                elif name in CONV_NAMES:
                    kinds.append("conv")
                else:
                    raise ConfigError(
                        f"layer_types[{i}] is {name!r}; known kinds: "
                        f"{', '.join(CONV_NAMES + ATTENTION_NAMES)}")
        elif has_any(data, ["full_attn_idxs"]):
            idxs = read_int_list(data, ["full_attn_idxs"])
            for i in idxs:
                if not 0 <= i < n_layers:
                    raise ConfigError(f"full_attn_idxs names layer {i} of {n_layers}")
            kinds = ["attention" if i in set(idxs) else "conv" for i in range(n_layers)]
        else:
            raise ConfigError("config.json has no layer_types / full_attn_idxs")
        if len(kinds) != n_layers:
            raise ConfigError(
                f"layer_types has {len(kinds)} entries but num_hidden_layers is {n_layers}")

        block_ff = read_int(data, ["block_ff_dim", "intermediate_size"], minimum=1)
        # ``block_ff_dim`` is the width before the adjustment, which is on unless the
        # key switches it off; a config that gives only ``intermediate_size`` and says
        # nothing about adjusting means that width itself.
        auto = read_bool(data, ["block_auto_adjust_ff_dim"], default=has_any(data, ["block_ff_dim"]))
        multiple_of = read_int(data, ["block_multiple_of", "multiple_of"],
                               default=256 if auto else None, minimum=1)
        multiplier = read_float(data, ["block_ffn_dim_multiplier"], default=None, positive=True)
        width = feed_forward_width(block_ff, auto, multiple_of, multiplier)

        eos = data.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else None
        return cls(
            architecture=str(archs[0]),
            hidden_size=hidden, num_layers=n_layers, num_heads=n_heads, num_kv_heads=n_kv,
            head_dim=head_dim, vocab_size=vocab, layer_types=tuple(kinds),
            block_ff_dim=block_ff, auto_adjust_ff_dim=auto, multiple_of=multiple_of,
            ffn_dim_multiplier=multiplier, intermediate_size=width,
            rope_theta=read_float(_with_nested_rope(data), ["rope_theta"], positive=True),
            norm_eps=read_float(data, ["norm_eps", "rms_norm_eps", "block_norm_eps"], positive=True),
            conv_L_cache=read_int(data, ["conv_L_cache"], minimum=1),
            conv_bias=read_bool(data, ["conv_bias"], default=False),
            tie_embedding=read_bool(data, ["tie_embedding", "tie_word_embeddings"], default=True),
            max_position_embeddings=read_int(data, ["max_position_embeddings"], default=0, minimum=0),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
        )

    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        out = {
            "architectures": [self.architecture],
            "model_type": "lfm2",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "layer_types": ["full_attention" if k == "attention" else "conv"
                            for k in self.layer_types],
            "block_ff_dim": self.block_ff_dim,
            "block_auto_adjust_ff_dim": self.auto_adjust_ff_dim,
            "rope_theta": self.rope_theta,
            "norm_eps": self.norm_eps,
            "conv_L_cache": self.conv_L_cache,
            "conv_bias": self.conv_bias,
            "tie_embedding": self.tie_embedding,
            "max_position_embeddings": self.max_position_embeddings,
        }
        if self.multiple_of is not None:
            out["block_multiple_of"] = self.multiple_of
        if self.ffn_dim_multiplier is not None:
            out["block_ffn_dim_multiplier"] = self.ffn_dim_multiplier
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out

    # ------------------------------------------------------------ translation
    def to_spec(self) -> ModelSpec:
        """Describe the model as parts.  Checkpoint names: the safetensors
        spelling first, then the reference's GGUF spelling
        (/root/reference/src/transformer/hybrid_layer.zig:300-315,
        hybrid_attn.zig:250-267, short_conv.zig:5-13, loader/gguf_model.zig:36-71)."""
        H, d = self.hidden_size, self.head_dim

        def names(hf: str, gguf: str) -> Tuple[str, ...]:
            return (hf, gguf)

        rope = PartSpec("rope", {"head_dim": d, "rotary_dim": d, "theta": self.rope_theta,
                                 "pairing": "half"})
        layers = []
        for i, kind in enumerate(self.layer_types):
            p, g = f"model.layers.{i}.", f"blk.{i}."
            if kind == "attention":
                mixer = PartSpec(
                    "gqa_attention",
                    {"hidden_size": H, "num_heads": self.num_heads,
                     "num_kv_heads": self.num_kv_heads, "head_dim": d,
                     "qk_norm": True, "norm_eps": self.norm_eps, "window": 0,
                     "softmax_scale": None, "bias": False, "position": rope},
                    {"q_proj.weight": names(p + "self_attn.q_proj.weight", g + "attn_q.weight"),
                     "k_proj.weight": names(p + "self_attn.k_proj.weight", g + "attn_k.weight"),
                     "v_proj.weight": names(p + "self_attn.v_proj.weight", g + "attn_v.weight"),
                     "out_proj.weight": names(p + "self_attn.out_proj.weight",
                                              g + "attn_output.weight"),
                     "q_norm.weight": names(p + "self_attn.q_layernorm.weight",
                                            g + "attn_q_norm.weight"),
                     "k_norm.weight": names(p + "self_attn.k_layernorm.weight",
                                            g + "attn_k_norm.weight")})
            else:
                tensors = {
                    "in_proj.weight": names(p + "conv.in_proj.weight",
                                            g + "shortconv.in_proj.weight"),
                    "conv.weight": names(p + "conv.conv.weight", g + "shortconv.conv.weight"),
                    "out_proj.weight": names(p + "conv.out_proj.weight",
                                             g + "shortconv.out_proj.weight"),
                }
                if self.conv_bias:
                    tensors.update({
                        "in_proj.bias": names(p + "conv.in_proj.bias", g + "shortconv.in_proj.bias"),
                        "conv.bias": names(p + "conv.conv.bias", g + "shortconv.conv.bias"),
                        "out_proj.bias": names(p + "conv.out_proj.bias",
                                               g + "shortconv.out_proj.bias"),
                    })
                mixer = PartSpec("short_conv",
                                 {"hidden_size": H, "kernel_size": self.conv_L_cache,
                                  "bias": self.conv_bias}, tensors)
            ffn = PartSpec(
                "swiglu", {"hidden_size": H, "intermediate_size": self.intermediate_size},
                {"gate.weight": names(p + "feed_forward.w1.weight", g + "ffn_gate.weight"),
                 "up.weight": names(p + "feed_forward.w3.weight", g + "ffn_up.weight"),
                 "down.weight": names(p + "feed_forward.w2.weight", g + "ffn_down.weight")})
            mixer_norm = PartSpec("rms_norm", {"width": H, "eps": self.norm_eps},
                                  {"weight": names(p + "operator_norm.weight",
                                                   g + "attn_norm.weight")})
            ffn_norm = PartSpec("rms_norm", {"width": H, "eps": self.norm_eps},
                                {"weight": names(p + "ffn_norm.weight", g + "ffn_norm.weight")})
            layers.append(LayerSpec.pre_norm(mixer, ffn, mixer_norm, ffn_norm))

        embedding = PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": H},
                             {"weight": ("model.embed_tokens.weight", "token_embd.weight")})
        final_norm = PartSpec("rms_norm", {"width": H, "eps": self.norm_eps},
                              {"weight": ("model.embedding_norm.weight", "token_embd_norm.weight",
                                          "output_norm.weight", "model.norm.weight")})
        lm_head = PartSpec("linear_head",
                           {"vocab_size": self.vocab_size, "hidden_size": H,
                            "tied": self.tie_embedding},
                           {} if self.tie_embedding else
                           {"weight": ("lm_head.weight", "output.weight")})
        schedule = tuple(LayerCall(i) for i in range(self.num_layers))
        # a tied checkpoint may still carry a copy of the head; it is not read
        ignored = ("lm_head.weight", "output.weight") if self.tie_embedding else ()
        return ModelSpec(self.architecture, H, self.vocab_size, embedding, tuple(layers),
                         schedule, final_norm, lm_head, self.max_position_embeddings, ignored)
