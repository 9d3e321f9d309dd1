"""Named shapes of the Llama 3 family as config.json dictionaries, for runs with random
weights: the command line's ``--random NAME`` and the benchmark take them from here (the
reference's example script names its model as a constant at its top, examples/infer.py:13-16,
and needs the checkpoint; here a name stands for the layer sizes alone).
"""
from __future__ import annotations

from typing import Dict, Tuple

LLAMA3_8B = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 4096,
    "num_hidden_layers": 32,
    "num_attention_heads": 32,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 14336,
    "vocab_size": 128256,
    "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": None,
    "max_position_embeddings": 8192,
    "tie_word_embeddings": False,
}
_LLAMA3_SCALING = {"rope_type": "llama3", "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                   "original_max_position_embeddings": 8192}
LLAMA32_3B = dict(LLAMA3_8B, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, intermediate_size=8192,
                  rope_scaling=dict(_LLAMA3_SCALING, factor=32.0), tie_word_embeddings=True)
LLAMA32_1B = dict(LLAMA3_8B, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32, head_dim=64, intermediate_size=8192,
                  rope_scaling=dict(_LLAMA3_SCALING, factor=32.0), tie_word_embeddings=True)
LLAMA31_70B = dict(LLAMA3_8B, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, intermediate_size=28672,
                   rope_scaling=dict(_LLAMA3_SCALING, factor=8.0))
# two shapes of a few thousand parameters that differ in every size and option
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 192, "vocab_size": 256, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "rope_scaling": None, "max_position_embeddings": 128, "tie_word_embeddings": False,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 128, "num_hidden_layers": 3, "num_attention_heads": 4,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 352, "vocab_size": 384, "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "max_position_embeddings": 256, "tie_word_embeddings": True,
}

# name -> (what to call it, config.json dictionary)
SHAPES: Dict[str, Tuple[str, dict]] = {
    "8b": ("Llama-3-8B", LLAMA3_8B),
    "3b": ("Llama-3.2-3B", LLAMA32_3B),
    "1b": ("Llama-3.2-1B", LLAMA32_1B),
    "70b": ("Llama-3.1-70B", LLAMA31_70B),
    "tiny-a": ("tiny Llama A", TINY_A),
    "tiny-b": ("tiny Llama B", TINY_B),
}


def shape(name: str) -> Tuple[str, dict]:
    if name not in SHAPES:
        raise ValueError(f"unknown shape {name!r}; known: {sorted(SHAPES)}")
    label, cfg = SHAPES[name]
    return label, dict(cfg)
