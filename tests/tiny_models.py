"""The tiny configurations the tests run on.  A and B differ in every size and
option: layers 2 / 3, kinds given by layer_types / by sliding_window_pattern,
window 8 / 5, hidden 64 / 96, heads 4:2 / 6:3, head size 16 / 32 (query width
equal to / different from hidden), intermediate 128 / 160, vocabulary 256 (a
power of two) / 509 (a prime), global base 1e6 / 5e5, no scaling / linear 4,
score scalar equal to / different from the head size, eps 1e-6 / 1e-5.
C has the head size of the large models (256), one key/value head and a
soft-cap.  D is not tiny in its layers: two layers with the attention sizes of
the 4B model (width 2560, heads 8:4 of 256, feed-forward 10240, window 1024,
global scaling 8) and
a vocabulary of 1003, for sequences that cross the window's edge; it is
written only by the tests that use it.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch

CONFIG_A = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 2,
    "layer_types": ["sliding_attention", "full_attention"],
    "hidden_size": 64,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "intermediate_size": 128,
    "vocab_size": 256,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 4096,
    "sliding_window": 8,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": None,
    "query_pre_attn_scalar": 16,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
    "attn_logit_softcapping": None,
}

CONFIG_B = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 3,
    "sliding_window_pattern": 3,
    "hidden_size": 96,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 32,
    "intermediate_size": 160,
    "vocab_size": 509,
    "rms_norm_eps": 1e-5,
    "max_position_embeddings": 2048,
    "sliding_window": 5,
    "rope_theta": 500000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 4.0},
    "query_pre_attn_scalar": 48,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}

CONFIG_C = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 2,
    "layer_types": ["full_attention", "sliding_attention"],
    "hidden_size": 80,
    "num_attention_heads": 2,
    "num_key_value_heads": 1,
    "head_dim": 256,
    "intermediate_size": 112,
    "vocab_size": 300,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 4096,
    "sliding_window": 70,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 8.0},
    "query_pre_attn_scalar": 256,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": 30.0,
}

CONFIG_D = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 2,
    "layer_types": ["sliding_attention", "full_attention"],
    "hidden_size": 2560,
    "num_attention_heads": 8,
    "num_key_value_heads": 4,
    "head_dim": 256,
    "intermediate_size": 10240,
    "vocab_size": 1003,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192,
    "sliding_window": 1024,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 8.0},
    "query_pre_attn_scalar": 256,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}

# The head geometry of the 27B model (32 query heads on 16 key/value heads of 128 dimensions, scores scaled by
# 168^-1/2, not by the head size) on a narrow layer: three layers, the global one in the middle.
CONFIG_E = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 3,
    "layer_types": ["sliding_attention", "full_attention", "sliding_attention"],
    "hidden_size": 672,
    "num_attention_heads": 32,
    "num_key_value_heads": 16,
    "head_dim": 128,
    "intermediate_size": 1344,
    "vocab_size": 811,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192,
    "sliding_window": 1024,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 8.0},
    "query_pre_attn_scalar": 168,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}

# The whole model at the sizes of Gemma 3 4B: 34 layers, every sixth one global, the full vocabulary.
CONFIG_4B = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 34,
    "sliding_window_pattern": 6,
    "hidden_size": 2560,
    "num_attention_heads": 8,
    "num_key_value_heads": 4,
    "head_dim": 256,
    "intermediate_size": 10240,
    "vocab_size": 262208,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 131072,
    "sliding_window": 1024,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 8.0},
    "query_pre_attn_scalar": 256,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}

# E's layers for sequences of many thousand tokens.
CONFIG_LONG = dict(CONFIG_E, max_position_embeddings=32768)

# Heads that the matrix-core attention kernels do not take, so that bf16 runs the kernel for any size too: a head
# size above 256 (and no multiple of 32), 17 query heads on each key/value head.
CONFIG_G = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 2,
    "layer_types": ["full_attention", "sliding_attention"],
    "hidden_size": 112,
    "num_attention_heads": 34,
    "num_key_value_heads": 2,
    "head_dim": 272,
    "intermediate_size": 200,
    "vocab_size": 333,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 1024,
    "sliding_window": 33,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 2.0},
    "query_pre_attn_scalar": 100,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}

CONFIGS = {"A": (CONFIG_A, 0), "B": (CONFIG_B, 1), "C": (CONFIG_C, 2)}
LARGER = {"D": (CONFIG_D, 3), "E": (CONFIG_E, 4), "4B": (CONFIG_4B, 5), "LONG": (CONFIG_LONG, 6), "G": (CONFIG_G, 7)}


def write_model(folder, name: str, dtype=torch.bfloat16, seed=None) -> Path:
    """Write config ``name`` with random weights into ``folder`` through the
    framework's random-weights mode; returns the folder."""
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401  (registers the architecture)
    from rvllm_amd.weights.random_init import write_random_model

    doc, default_seed = CONFIGS[name] if name in CONFIGS else LARGER[name]
    arch = architecture_of(doc)
    config = arch.read_config(doc, f"tiny config {name}")
    out = write_random_model(Path(folder), config, default_seed if seed is None else seed, dtype)
    # keep the document as written above, so that each spelling of the keys is read
    (out / "config.json").write_text(json.dumps(doc, indent=2))
    return out
