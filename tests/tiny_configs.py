"""Tiny Llama configurations for tests, as config.json dicts.  A and B are the two
the build brief names; they differ in every size and option.  C has a head size the
matrix-core attention kernel takes (64) with a hidden size and vocabulary that are no
powers of two; D has head size 128, more than 16 query heads per kv head's worth of
variety (8 per kv head) and a long-context scaling.
"""

TINY_A = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "intermediate_size": 192,
    "vocab_size": 256,
    "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0,
    "rope_scaling": None,
    "max_position_embeddings": 128,
    "tie_word_embeddings": False,
    "hidden_act": "silu",
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 128,
    "num_hidden_layers": 3,
    "num_attention_heads": 4,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "intermediate_size": 352,
    "vocab_size": 384,
    "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 64,
    },
    "max_position_embeddings": 256,
    "tie_word_embeddings": True,
    "hidden_act": "silu",
}

TINY_C = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 192,
    "num_hidden_layers": 2,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 64,
    "intermediate_size": 328,
    "vocab_size": 515,
    "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0,
    "max_position_embeddings": 512,
    "tie_word_embeddings": False,
}

TINY_D = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 320,
    "num_hidden_layers": 2,
    "num_attention_heads": 8,
    "num_key_value_heads": 1,
    "head_dim": 128,
    "intermediate_size": 520,
    "vocab_size": 1000,
    "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 32.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 128,
    },
    "max_position_embeddings": 1024,
    "tie_word_embeddings": True,
}

# Sizes that meet none of the fast paths: a head size the matrix-core attention does not take
# (48), three query heads on one kv head, a hidden size that differs from heads x head size,
# widths that are no multiples of 8 (no 16-byte rows: the few-row matrix-core product and the
# packed gate/up layout do not apply), one layer, an odd vocabulary.
TINY_E = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 100,
    "num_hidden_layers": 1,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "head_dim": 48,
    "intermediate_size": 90,
    "vocab_size": 1001,
    "rms_norm_eps": 3e-6,
    "rope_theta": 25000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 4.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 2.0,
        "original_max_position_embeddings": 32,
    },
    "max_position_embeddings": 192,
    "tie_word_embeddings": True,
}

# Three query heads on each of two kv heads at head size 128 (the head layout of Llama-3.2-3B):
# with pages of 64 tokens the matrix-core attention runs over tiled pages with tiles of
# 5 tokens x 3 heads, one column of every wave standing for nothing.
TINY_F = {
    "architectures": ["LlamaForCausalLM"],
    "model_type": "llama",
    "hidden_size": 264,
    "num_hidden_layers": 2,
    "num_attention_heads": 6,
    "num_key_value_heads": 2,
    "head_dim": 128,
    "intermediate_size": 392,
    "vocab_size": 777,
    "rms_norm_eps": 2e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 32.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 96,
    },
    "max_position_embeddings": 768,
    "tie_word_embeddings": True,
}

ALL = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}
