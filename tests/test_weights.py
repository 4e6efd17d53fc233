"""Safetensors I/O, loading by name with one clear error, kept precisions, and
the random model writer."""

import json
import os
import struct

import pytest
import torch

from tiny_configs import TINY_A, TINY_B
from zig_ai_amd.config import config_from_dict
from zig_ai_amd.weights import (Checkpoint, SafetensorsError, WeightError, expected_tensors,
                                keep_dtype, load_tensors, random_tensors, write_random_model,
                                write_safetensors)


def test_safetensors_round_trip_against_the_library(tmp_path):
    from safetensors.torch import load_file, save_file
    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int64),
               "c": torch.randn(2, 2, 2), "d": torch.tensor(3.5)}
    ours = str(tmp_path / "model.safetensors")
    write_safetensors(ours, tensors, {"who": "us"})
    theirs = load_file(ours)                       # the library reads what we write
    for k, v in tensors.items():
        assert torch.equal(theirs[k], v)
    os.remove(ours)
    save_file(tensors, ours)                       # and we read what the library writes
    ck = Checkpoint(str(tmp_path))
    assert sorted(ck.names()) == ["a", "b", "c", "d"]
    for k, v in tensors.items():
        assert torch.equal(ck.tensor(k), v) and ck.shape(k) == tuple(v.shape)


def test_safetensors_offsets_count_from_the_data_section(tmp_path):
    """Offsets are relative to the byte after the header (8 + header length)."""
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, {"x": torch.tensor([1.0, 2.0]), "y": torch.tensor([3.0])})
    raw = open(path, "rb").read()
    (n,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + n])
    begin, end = header["y"]["data_offsets"]
    assert struct.unpack("<f", raw[8 + n + begin:8 + n + end])[0] == 3.0


def test_truncated_and_malformed_files(tmp_path):
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, {"x": torch.randn(64)})
    raw = open(path, "rb").read()
    open(path, "wb").write(raw[:-10])
    with pytest.raises(SafetensorsError, match="truncated"):
        Checkpoint(str(tmp_path))
    open(path, "wb").write(raw[:4])
    with pytest.raises(SafetensorsError, match="shorter"):
        Checkpoint(str(tmp_path))
    open(path, "wb").write(struct.pack("<Q", 5) + b"{bad}")
    with pytest.raises(SafetensorsError, match="JSON"):
        Checkpoint(str(tmp_path))
    os.remove(path)
    with pytest.raises(SafetensorsError, match="neither"):
        Checkpoint(str(tmp_path))


def test_sharded_checkpoint(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    ck = Checkpoint(str(tmp_path))
    assert torch.equal(ck.tensor("a"), torch.ones(2)) and ck.shape("b") == (3,)


def test_random_model_is_reproducible_and_loads(tmp_path):
    d1, d2, d3 = (str(tmp_path / n) for n in "abc")
    write_random_model(TINY_B, d1, seed=1, dtype=torch.bfloat16)
    write_random_model(TINY_B, d2, seed=1, dtype=torch.bfloat16)
    write_random_model(TINY_B, d3, seed=2, dtype=torch.bfloat16)
    c1, c2, c3 = Checkpoint(d1), Checkpoint(d2), Checkpoint(d3)
    assert sorted(c1.names()) == sorted(c2.names())
    same = [torch.equal(c1.tensor(n), c2.tensor(n)) for n in c1.names()]
    assert all(same)
    assert not torch.equal(c1.tensor("model.embed_tokens.weight"), c3.tensor("model.embed_tokens.weight"))
    assert json.load(open(os.path.join(d1, "config.json"))) == TINY_B
    # what the architecture needs, under the names checkpoints use
    names = set(c1.names())
    assert {"model.embed_tokens.weight", "model.embedding_norm.weight", "lm_head.weight",
            "model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.q_layernorm.weight",
            "model.layers.1.conv.in_proj.weight", "model.layers.1.conv.conv.weight",
            "model.layers.1.conv.conv.bias", "model.layers.1.conv.out_proj.weight",
            "model.layers.1.operator_norm.weight", "model.layers.1.ffn_norm.weight",
            "model.layers.1.feed_forward.w1.weight", "model.layers.1.feed_forward.w2.weight",
            "model.layers.1.feed_forward.w3.weight"} <= names
    assert c1.shape("model.layers.1.conv.conv.weight") == (96, 1, 4)
    assert c1.shape("model.layers.1.feed_forward.w1.weight") == (256, 96)
    emb = c1.tensor("model.embed_tokens.weight").float()
    assert abs(float(emb.std()) - 0.02) < 0.002 and abs(float(emb.mean())) < 0.002
    assert torch.equal(c1.tensor("model.embedding_norm.weight").float(), torch.ones(96))
    spec = config_from_dict(TINY_B).to_spec()
    loaded = load_tensors(d1, spec, torch.bfloat16, "cpu")
    assert loaded[("layer", 1, "mixer")]["conv.weight"].shape == (96, 4)
    assert loaded[("layer", 1, "mixer")]["conv.weight"].dtype == torch.float32
    assert loaded[("layer", 0, "mixer")]["q_proj.weight"].dtype == torch.bfloat16
    assert loaded[("layer", 0, "mixer_norm")]["weight"].dtype == torch.float32
    wide = load_tensors(d1, spec, torch.float32, "cpu")
    assert wide[("layer", 0, "mixer")]["q_proj.weight"].dtype == torch.float32
    assert torch.equal(wide[("layer", 0, "mixer")]["q_proj.weight"],
                       loaded[("layer", 0, "mixer")]["q_proj.weight"].float())


def test_random_values_are_keyed_by_seed_name_and_index(tmp_path):
    """A value is a function of (seed, tensor name, element index): the known answer of the
    generator's round function, prefixes and chunks agree, and a tensor does not change
    when the model around it does (more layers: other tensors are drawn before it)."""
    from zig_ai_amd.weights import random_init as ri
    # Philox-4x32-10, counter 0, key 0: the generator's published known answer
    words = ri._philox(torch.zeros(1, dtype=torch.int64), (0, 0))
    assert [int(w[0]) for w in words] == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    a = ri.keyed_normal(7, "x.weight", 1003)
    assert torch.equal(a[:99], ri.keyed_normal(7, "x.weight", 99))
    assert torch.equal(a, ri.keyed_normal(7, "x.weight", 1003, chunk=64))
    assert not torch.equal(a, ri.keyed_normal(8, "x.weight", 1003))
    assert not torch.equal(a, ri.keyed_normal(7, "y.weight", 1003))
    big = ri.keyed_normal(1, "t", 400000)
    assert abs(float(big.mean())) < 0.01 and abs(float(big.std()) - 1) < 0.01
    assert abs(float((big.abs() > 2).float().mean()) - 0.0455) < 0.003
    deeper = dict(TINY_A, num_hidden_layers=5,
                  layer_types=["full_attention"] + TINY_A["layer_types"])
    d1, d2 = str(tmp_path / "a"), str(tmp_path / "b")
    write_random_model(TINY_A, d1, seed=3, dtype=torch.float32)
    write_random_model(deeper, d2, seed=3, dtype=torch.float32)
    c1, c2 = Checkpoint(d1), Checkpoint(d2)
    for name in ("model.embed_tokens.weight", "model.layers.1.conv.in_proj.weight",
                 "model.layers.3.feed_forward.w2.weight"):
        assert torch.equal(c1.tensor(name), c2.tensor(name)), name


@pytest.mark.gpu
def test_a_random_model_drawn_on_the_gpu_is_the_folder(tmp_path):
    """``DecoderModel.from_random`` (what the benchmark builds) holds the tensors that the
    random model writer stores for the same configuration and seed, drawn on the CPU."""
    from zig_ai_amd.engine import DecoderModel
    from zig_ai_amd.weights import random_init as ri
    folder = str(tmp_path / "m")
    tensors = ri.random_tensors(config_from_dict(TINY_B).to_spec(), 11, torch.bfloat16,
                                norm_init="around_one", device="cpu")
    ri.write_random_model(TINY_B, folder, seed=11, dtype=torch.bfloat16, norm_init="around_one")
    stored = Checkpoint(folder)
    for name, t in tensors.items():
        assert torch.equal(stored.tensor(name), t), name
    drawn = DecoderModel.from_random(TINY_B, seed=11, dtype="bfloat16", norm_init="around_one")
    loaded = DecoderModel.from_folder(folder, "bfloat16")
    for a, b in zip(drawn.blocks, loaded.blocks):
        for part in ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm"):
            pa, pb = getattr(a, part), getattr(b, part)
            for key, value in vars(pa).items():
                if isinstance(value, torch.Tensor):
                    assert torch.equal(value, getattr(pb, key)), (part, key)
    assert torch.equal(drawn.embedding.weight, loaded.embedding.weight)
    assert torch.equal(drawn.head.weight, loaded.head.weight)


def test_kept_precision():
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert keep_dtype(bf, "matrix", bf) == bf
    assert keep_dtype(f32, "matrix", bf) == f32          # stored in 32-bit: stays so
    assert keep_dtype(f16, "matrix", bf) == f32
    assert keep_dtype(bf, "matrix", f32) == f32
    assert keep_dtype(bf, "norm", bf) == f32
    assert keep_dtype(torch.int64, "table", bf) == torch.int32


def test_one_error_lists_everything(tmp_path):
    spec = config_from_dict(TINY_A).to_spec()
    tensors = random_tensors(spec, seed=0, dtype=torch.bfloat16)
    del tensors["model.layers.2.self_attn.k_proj.weight"]
    del tensors["model.embedding_norm.weight"]
    tensors["model.layers.9.surprise.weight"] = torch.zeros(2)
    tensors["lm_head.weight"] = torch.zeros(256, 64)                      # tied: present, not read
    tensors["model.layers.0.conv.in_proj.weight"] = torch.zeros(100, 64)  # should be [192, 64]
    tensors["model.layers.1.ffn_norm.weight"] = torch.zeros(64, dtype=torch.float64)
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        load_tensors(str(tmp_path), spec, torch.bfloat16, "cpu")
    err = e.value
    assert err.missing == ["model.layers.2.self_attn.k_proj.weight", "model.embedding_norm.weight"]
    assert err.unexpected == ["model.layers.9.surprise.weight"]   # a tied head's copy is ignored
    assert len(err.wrong_shape) == 1 and "[100, 64]" in err.wrong_shape[0] and "[192, 64]" in err.wrong_shape[0]
    assert err.wrong_dtype == ["model.layers.1.ffn_norm.weight: F64"]
    text = str(err)
    for piece in ("missing (2)", "unexpected (1)", "wrong shape (1)", "unsupported dtype (1)"):
        assert piece in text


def test_reference_spelling_of_names_is_accepted(tmp_path):
    """The GGUF-style names of the reference (hybrid_layer.zig:300-315) load too."""
    spec = config_from_dict(TINY_A).to_spec()
    tensors = {}
    for exp in expected_tensors(spec):
        t = torch.zeros(exp.rule.stored_shape or exp.rule.shapes[0], dtype=torch.bfloat16)
        tensors[exp.names[1]] = t
    assert "blk.2.attn_q.weight" in tensors and "token_embd.weight" in tensors
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    loaded = load_tensors(str(tmp_path), spec, torch.bfloat16, "cpu")
    assert ("layer", 2, "mixer") in loaded


def test_optional_projection_biases(tmp_path):
    """conv_bias: the convolution's bias is required, the projections' are used if there."""
    spec = config_from_dict(TINY_B).to_spec()
    tensors = random_tensors(spec, seed=0)
    for i in (1, 2, 4):
        del tensors[f"model.layers.{i}.conv.in_proj.bias"]
        del tensors[f"model.layers.{i}.conv.out_proj.bias"]
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    loaded = load_tensors(str(tmp_path), spec, torch.bfloat16, "cpu")
    assert "in_proj.bias" not in loaded[("layer", 1, "mixer")]
    del tensors["model.layers.1.conv.conv.bias"]
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    with pytest.raises(WeightError, match="conv.conv.bias"):
        load_tensors(str(tmp_path), spec, torch.bfloat16, "cpu")
