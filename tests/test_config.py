"""Configuration parsing, the feed-forward width rule, the registry."""

import json

import pytest

from tiny_configs import TINY_A, TINY_B, TINY_C
from zig_ai_amd.config import (ConfigError, Lfm2Config, config_from_dict, feed_forward_width,
                               known_architectures, load_config, register_architecture)


def test_ffn_width_rule():
    # the sizes of the three real shapes and of tiny-B
    assert feed_forward_width(12288, True, 256, 1.0) == 8192
    assert feed_forward_width(6656, True, 256, 1.0) == 4608
    assert feed_forward_width(10752, True, 256, None) == 7168
    assert feed_forward_width(384, True, 128, None) == 256
    assert feed_forward_width(192, False, None, None) == 192
    assert feed_forward_width(200, True, 8, 1.3) == 176
    with pytest.raises(ConfigError):
        feed_forward_width(384, True, None, None)


def test_tiny_configs_parse():
    a, b, c = (config_from_dict(x) for x in (TINY_A, TINY_B, TINY_C))
    assert isinstance(a, Lfm2Config)
    assert (a.hidden_size, a.num_heads, a.num_kv_heads, a.head_dim) == (64, 4, 2, 16)
    assert a.layer_types == ("conv", "conv", "attention", "conv")
    assert a.intermediate_size == 192 and a.tie_embedding and not a.conv_bias
    assert (b.head_dim, b.intermediate_size, b.conv_L_cache, b.norm_eps) == (32, 256, 4, 1e-6)
    assert not b.tie_embedding and b.conv_bias and b.rope_theta == 1e6
    assert c.head_dim == 48 and c.intermediate_size == 176
    # every size and option differs between A and B
    for f in ("hidden_size", "num_layers", "num_heads", "num_kv_heads", "head_dim", "vocab_size",
              "intermediate_size", "rope_theta", "norm_eps", "conv_L_cache", "conv_bias",
              "tie_embedding", "auto_adjust_ff_dim"):
        assert getattr(a, f) != getattr(b, f), f


def test_round_trip_and_aliases():
    a = config_from_dict(TINY_B)
    assert config_from_dict(a.to_dict()) == a
    alt = dict(TINY_A)
    del alt["layer_types"]
    alt["full_attn_idxs"] = [2]
    alt["tie_word_embeddings"] = alt.pop("tie_embedding")
    assert config_from_dict(alt).layer_types == config_from_dict(TINY_A).layer_types
    alt2 = dict(TINY_A, layer_types=["short_conv", "conv", "attention", "conv"])
    assert config_from_dict(alt2).layer_types == config_from_dict(TINY_A).layer_types


@pytest.mark.parametrize("change,match", [
    ({"hidden_size": None}, "hidden_size"),
    ({"rope_theta": None}, "rope_theta"),
    ({"norm_eps": None}, "norm_eps"),
    ({"conv_L_cache": None}, "conv_L_cache"),
    ({"layer_types": None}, "layer_types"),
    ({"layer_types": ["conv"]}, "4"),
    ({"layer_types": ["conv", "conv", "mamba", "conv"]}, "mamba"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_size": 66}, "head_dim"),
    ({"vocab_size": "many"}, "integer"),
    ({"conv_bias": 1}, "true or false"),
    ({"norm_eps": -1.0}, "positive"),
    ({"architectures": ["GptForCausalLM"]}, "Lfm2ForCausalLM"),
    ({"architectures": None}, "architectures"),
])
def test_config_errors(change, match):
    bad = dict(TINY_A)
    for k, v in change.items():
        if v is None:
            bad.pop(k, None)
        else:
            bad[k] = v
    with pytest.raises(ConfigError, match=match):
        config_from_dict(bad)


def test_defaults_of_the_width_keys():
    only_width = {k: v for k, v in TINY_A.items() if not k.startswith("block_")}
    only_width["intermediate_size"] = 192
    assert config_from_dict(only_width).intermediate_size == 192          # taken as it is
    pre = dict(only_width, block_ff_dim=12288)
    del pre["intermediate_size"]
    assert config_from_dict(pre).intermediate_size == 8192                # adjusted, multiple of 256
    nested = {k: v for k, v in TINY_A.items() if k != "rope_theta"}
    nested["rope_parameters"] = {"rope_theta": 12345.0, "rope_type": "default"}
    assert config_from_dict(nested).rope_theta == 12345.0


def test_load_config_from_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert load_config(str(tmp_path)).hidden_size == 64
    with pytest.raises(ConfigError, match="does not exist"):
        load_config(str(tmp_path / "nowhere"))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))


def test_registry():
    assert "Lfm2ForCausalLM" in known_architectures()

    class Other:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_spec(self):
            return None

    register_architecture("OtherForCausalLM", Other)
    assert isinstance(config_from_dict({"architectures": ["OtherForCausalLM"]}), Other)
    with pytest.raises(TypeError):
        register_architecture("Broken", object)


def test_spec_of_lfm2():
    spec = config_from_dict(TINY_B).to_spec()
    assert [l.mixer.kind for l in spec.layers] == [
        "gqa_attention", "short_conv", "short_conv", "gqa_attention", "short_conv", "gqa_attention"]
    assert [c.layer for c in spec.schedule] == list(range(6))
    assert spec.lm_head.tensors["weight"][0] == "lm_head.weight"
    assert config_from_dict(TINY_A).to_spec().lm_head.tensors == {}
    att = spec.layers[0].mixer.params
    assert att["position"].kind == "rope" and att["position"].params["theta"] == 1e6
    assert spec.layers[1].mixer.params["kernel_size"] == 4
