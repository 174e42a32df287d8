"""Tiny configurations and weight makers for the tests (never the product's own)."""
from __future__ import annotations

import zlib

import numpy as np

# 2 layers, grouped heads (g=2), adjacent-pair rotation, no frequency scaling, tied head.
TINY_A = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 64,
    "intermediate_size": 192,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "vocab_size": 256,
    "max_position_embeddings": 128,
    "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0,
    "rope_scaling": None,
    "rope_pairing": "adjacent",
    "tie_word_embeddings": True,
    "hidden_act": "silu",
}

# 3 layers, one kv head for 3 query heads, half-split rotation (the default), llama3
# scaling whose three branches are all hit at head_dim 32, another eps, separate head.
TINY_B = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 96,
    "intermediate_size": 320,
    "num_hidden_layers": 3,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "vocab_size": 384,
    "max_position_embeddings": 256,
    "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 64,
    },
    "tie_word_embeddings": False,
    "hidden_act": "silu",
}

# The head size and grouping of the shape that bench.py measures (head_dim 64, four query heads to
# a kv head), so that the kernels built for it are also checked inside a whole model; tied head,
# a width and a vocabulary that no tile divides.
TINY_D = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 136,
    "intermediate_size": 264,
    "num_hidden_layers": 2,
    "num_attention_heads": 8,
    "num_key_value_heads": 2,
    "head_dim": 64,
    "vocab_size": 515,
    "max_position_embeddings": 512,
    "rms_norm_eps": 2e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 32.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 128,
    },
    "tie_word_embeddings": True,
    "hidden_act": "silu",
}

# Sizes that are no power of two anywhere: head_dim 48 with heads*head_dim != hidden,
# as many kv heads as heads, a vocabulary that no tile divides, a longer context.
TINY_C = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 112,
    "intermediate_size": 200,
    "num_hidden_layers": 2,
    "num_attention_heads": 5,
    "num_key_value_heads": 5,
    "head_dim": 48,
    "vocab_size": 1000,
    "max_position_embeddings": 1024,
    "rms_norm_eps": 1e-5,
    "rope_theta": 50000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 4.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 2.0,
        "original_max_position_embeddings": 256,
    },
    "tie_word_embeddings": False,
    "hidden_act": "silu",
}


def dims(cfg):
    d = cfg["hidden_size"]
    H = cfg["num_attention_heads"]
    K = cfg.get("num_key_value_heads", H)
    hs = cfg.get("head_dim") or d // H
    return d, H, K, hs, cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]


def tensor_shapes(cfg):
    d, H, K, hs, F, V, L = dims(cfg)
    shapes = {"model.embed_tokens.weight": (V, d), "model.norm.weight": (d,)}
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (V, d)
    for i in range(L):
        p = f"model.layers.{i}."
        shapes[p + "input_layernorm.weight"] = (d,)
        shapes[p + "self_attn.q_proj.weight"] = (H * hs, d)
        shapes[p + "self_attn.k_proj.weight"] = (K * hs, d)
        shapes[p + "self_attn.v_proj.weight"] = (K * hs, d)
        shapes[p + "self_attn.o_proj.weight"] = (d, H * hs)
        shapes[p + "post_attention_layernorm.weight"] = (d,)
        shapes[p + "mlp.gate_proj.weight"] = (F, d)
        shapes[p + "mlp.up_proj.weight"] = (F, d)
        shapes[p + "mlp.down_proj.weight"] = (d, F)
    return shapes


def make_weights(cfg, seed, std=0.02, norm_std=0.0):
    """float32 numpy weights: matrices N(0, std), norm weights 1 + N(0, norm_std)."""
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
        if len(shape) == 1:
            out[name] = (1.0 + norm_std * rng.standard_normal(shape)).astype(np.float32)
        else:
            out[name] = (std * rng.standard_normal(shape)).astype(np.float32)
    return out


def tokens(cfg, seed, n):
    rng = np.random.default_rng([seed, 77])
    return rng.integers(0, cfg["vocab_size"], size=n).tolist()
