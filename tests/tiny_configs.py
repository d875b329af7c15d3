"""Tiny Llama configurations for tests.  A and B differ in every size and option; C adds a
sliding window on some layers, a partial rotary width, linear rotary scaling and biases; D has heads
of 64 (the head size of the 128-row prompt attention kernel) and room for a thousand positions, so that
a portion of a prompt meets contexts of many key tiles; E has heads of 64 with a sliding window on two of its three
layers, so that the matrix-core attention kernels meet windows, pages that were given back (table entries of -1)
and pages that are used again; F has heads of 128, one key/value head and `yarn` scaling over four times its original
context; G has as many key/value heads as heads, a partial rotary width and `longrope` scaling whose long factors apply."""
import json

import numpy as np
import torch

TINY_A = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "intermediate_size": 176, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 128, "hidden_act": "silu",
}
TINY_B = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 3, "hidden_size": 160, "num_attention_heads": 5, "num_key_value_heads": 1, "head_dim": 32,
    "intermediate_size": 432, "vocab_size": 512, "rope_theta": 500000.0, "rms_norm_eps": 1e-6,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "tie_word_embeddings": True, "max_position_embeddings": 256, "hidden_act": "silu",
}
TINY_C = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 4, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48,
    "intermediate_size": 200, "vocab_size": 300, "rope_theta": 50000.0, "rms_norm_eps": 3e-6,
    "rope_scaling": {"rope_type": "linear", "factor": 2.0}, "partial_rotary_factor": 0.5,
    "sliding_window": 24, "layer_types": ["sliding_attention", "full_attention", "sliding_attention", "full_attention"],
    "tie_word_embeddings": False, "max_position_embeddings": 192, "hidden_act": "silu",
}
TINY_D = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
    "intermediate_size": 320, "vocab_size": 384, "rope_theta": 100000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 256},
    "tie_word_embeddings": False, "max_position_embeddings": 1024, "hidden_act": "silu",
}
TINY_E = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64,
    "intermediate_size": 272, "vocab_size": 320, "rope_theta": 250000.0, "rms_norm_eps": 2e-6,
    "sliding_window": 40, "layer_types": ["sliding_attention", "full_attention", "sliding_attention"],
    "tie_word_embeddings": True, "max_position_embeddings": 512, "hidden_act": "silu",
}
TINY_F = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 144, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 128,
    "intermediate_size": 208, "vocab_size": 272, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": {"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64, "beta_fast": 16.0,
                     "beta_slow": 2.0},
    "tie_word_embeddings": False, "max_position_embeddings": 256, "hidden_act": "silu",
}
TINY_G = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 4, "num_key_value_heads": 4, "head_dim": 32,
    "intermediate_size": 144, "vocab_size": 200, "rope_theta": 20000.0, "rms_norm_eps": 1e-6,
    "partial_rotary_factor": 0.75,
    "rope_scaling": {"rope_type": "longrope", "original_max_position_embeddings": 48,
                     "short_factor": [1.0, 1.0, 1.05, 1.1, 1.2, 1.3, 1.4, 1.5, 1.6, 1.7, 1.8, 1.9],
                     "long_factor": [1.0, 1.1, 1.3, 1.6, 2.0, 2.4, 2.8, 3.0, 3.2, 3.3, 3.4, 3.5]},
    "tie_word_embeddings": True, "max_position_embeddings": 160, "hidden_act": "silu",
}
PAGE_SIZES = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 16, "F": 32, "G": 8}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F, "G": TINY_G}


def to_float64(tensors):
    """Checkpoint tensors (torch, any float type) as float64 NumPy arrays for the plain implementation."""
    return {n: t.to(torch.float64).numpy() for n, t in tensors.items()}


def random_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()
