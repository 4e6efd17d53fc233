"""Small LFM2 configurations for tests.  A and B are the two that differ in
every size and option; C adds sizes that are multiples of neither 16 nor a
power of two where the kernels allow it."""

TINY_A = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 64, "num_hidden_layers": 4, "num_attention_heads": 4,
    "num_key_value_heads": 2, "vocab_size": 256,
    "layer_types": ["conv", "conv", "full_attention", "conv"],
    "block_ff_dim": 192, "block_auto_adjust_ff_dim": False,
    "rope_theta": 10000.0, "norm_eps": 1e-5, "conv_L_cache": 3, "conv_bias": False,
    "tie_embedding": True, "max_position_embeddings": 4096,
}

TINY_B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 96, "num_hidden_layers": 6, "num_attention_heads": 3,
    "num_key_value_heads": 1, "head_dim": 32, "vocab_size": 512,
    "layer_types": ["full_attention", "conv", "conv", "full_attention", "conv", "full_attention"],
    "block_ff_dim": 384, "block_auto_adjust_ff_dim": True, "block_multiple_of": 128,
    "rope_theta": 1000000.0, "norm_eps": 1e-6, "conv_L_cache": 4, "conv_bias": True,
    "tie_embedding": False, "max_position_embeddings": 4096,
}

TINY_C = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 80, "num_hidden_layers": 3, "num_attention_heads": 5,
    "num_key_value_heads": 5, "head_dim": 48, "vocab_size": 301,
    "layer_types": ["full_attention", "conv", "full_attention"],
    "block_ff_dim": 200, "block_auto_adjust_ff_dim": True, "block_multiple_of": 8,
    "block_ffn_dim_multiplier": 1.3,
    "rope_theta": 50000.0, "norm_eps": 3e-6, "conv_L_cache": 2, "conv_bias": True,
    "tie_embedding": True, "max_position_embeddings": 4096,
}

# sizes the matrix-core attention kernel takes (head_dim 64, four query heads per group)
TINY_D = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 128, "num_hidden_layers": 3, "num_attention_heads": 8,
    "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 384,
    "layer_types": ["full_attention", "conv", "full_attention"],
    "block_ff_dim": 320, "block_auto_adjust_ff_dim": False,
    "rope_theta": 1000000.0, "norm_eps": 1e-5, "conv_L_cache": 3, "conv_bias": False,
    "tie_embedding": True, "max_position_embeddings": 4096,
}

# head_dim 128 on the matrix-core attention kernels, three query heads per group, a
# head width that is not the hidden size's share
TINY_F = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 192, "num_hidden_layers": 2, "num_attention_heads": 3,
    "num_key_value_heads": 1, "head_dim": 128, "vocab_size": 520,
    "layer_types": ["conv", "full_attention"],
    "intermediate_size": 264,
    "rope_theta": 100000.0, "norm_eps": 2e-5, "conv_L_cache": 4, "conv_bias": True,
    "tie_embedding": False, "max_position_embeddings": 2048,
}

# a wide, deep one: five layers, four of them attention on the matrix cores, width 1536 (the
# decode kernels that run the norm themselves take it).  Of 3,000 configurations drawn at
# random this one had the largest end-to-end deviation in bfloat16 (2.6e-2 of the largest
# logit, with 6.7e-6 in 32-bit: rounding, not logic).
TINY_G = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 1536, "num_hidden_layers": 5, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 417,
    "layer_types": ["full_attention", "full_attention", "full_attention", "conv", "full_attention"],
    "intermediate_size": 176, "rope_theta": 1000000.0, "norm_eps": 1e-6, "conv_L_cache": 3,
    "conv_bias": False, "tie_embedding": False, "max_position_embeddings": 4096,
}

# two layers at the sizes of the LFM2-1.2B shape: the kernels' large-size paths
REAL_2L = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 2048, "num_hidden_layers": 2, "num_attention_heads": 32,
    "num_key_value_heads": 8, "vocab_size": 65536, "layer_types": ["conv", "full_attention"],
    "block_ff_dim": 12288, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
    "block_ffn_dim_multiplier": 1.0, "rope_theta": 1000000.0, "norm_eps": 1e-5,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 128000,
}

# three layers (ShortConv, attention, ShortConv) at the same sizes, for whole requests of
# hundreds of tokens under every way of cutting them
REAL_3L = dict(REAL_2L, num_hidden_layers=3, layer_types=["conv", "full_attention", "conv"])

# two layers at the LFM2-350M shape's sizes (hidden 1024, two query heads per key/value
# head, feed-forward 6656 -> 4608) and at the LFM2-2.6B shape's feed-forward width
# (10752 -> 7168): the sizes the other measured shapes add to the 1.2B shape's
REAL_350M_2L = dict(REAL_2L, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                    block_ff_dim=6656)
REAL_26B_2L = dict(REAL_2L, block_ff_dim=10752)

# widths that are multiples of neither 8 nor 16: fine in 32-bit, refused in bfloat16
TINY_E = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 60, "num_hidden_layers": 2, "num_attention_heads": 3,
    "num_key_value_heads": 3, "head_dim": 16, "vocab_size": 131,
    "layer_types": ["conv", "full_attention"],
    "intermediate_size": 100,
    "rope_theta": 10000.0, "norm_eps": 1e-5, "conv_L_cache": 5, "conv_bias": False,
    "tie_embedding": True, "max_position_embeddings": 512,
}
