"""Test-only helpers: the tiny configurations and a weight generator of the tests' own."""

from __future__ import annotations

import torch

# Two tiny Qwen3 configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 256, "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "max_position_embeddings": 128, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
    "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "bos_token_id": 1, "eos_token_id": 2,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 331, "hidden_size": 96, "intermediate_size": 160, "num_hidden_layers": 3,
    "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 32,
    "max_position_embeddings": 512, "rms_norm_eps": 1e-5, "rope_theta": 1000000.0,
    "hidden_act": "silu", "attention_bias": True, "attention_dropout": 0.0,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "bos_token_id": 0, "eos_token_id": [5, 7],
}
# Heads of 64 dims, the smallest the decode attention kernel rotates itself; three query heads per
# kv head, and every other size unlike A and B again.
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "vocab_size": 300, "hidden_size": 80, "intermediate_size": 176, "num_hidden_layers": 2,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64,
    "max_position_embeddings": 640, "rms_norm_eps": 3e-6, "rope_theta": 500000.0,
    "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "bos_token_id": 3, "eos_token_id": 4,
}


def qwen3_tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a dense Qwen3 checkpoint (reference mini_llm/checkpoint.py:287-344)."""
    h, i, d = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    shapes = {"model.embed_tokens.weight": (cfg["vocab_size"], h), "model.norm.weight": (h,)}
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (cfg["vocab_size"], h)
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        shapes.update({
            f"{p}.input_layernorm.weight": (h,), f"{p}.post_attention_layernorm.weight": (h,),
            f"{p}.self_attn.q_norm.weight": (d,), f"{p}.self_attn.k_norm.weight": (d,),
            f"{p}.self_attn.q_proj.weight": (nq * d, h), f"{p}.self_attn.k_proj.weight": (nkv * d, h),
            f"{p}.self_attn.v_proj.weight": (nkv * d, h), f"{p}.self_attn.o_proj.weight": (h, nq * d),
            f"{p}.mlp.gate_proj.weight": (i, h), f"{p}.mlp.up_proj.weight": (i, h),
            f"{p}.mlp.down_proj.weight": (h, i),
        })
        if cfg.get("attention_bias", False):
            shapes.update({
                f"{p}.self_attn.q_proj.bias": (nq * d,), f"{p}.self_attn.k_proj.bias": (nkv * d,),
                f"{p}.self_attn.v_proj.bias": (nkv * d,),
            })
    return shapes


def random_qwen3_weights(cfg: dict, seed: int, dtype=torch.float32) -> dict:
    """Weights whose every part contributes at order one, rounded to bfloat16 values.

    Matrices N(0, 1/fan_in), embedding N(0, 1), norm weights 1 + N(0, 0.1), biases N(0, 0.1):
    with the usual N(0, 0.02) the feed-forward would add about 1e-4 of the residual
    and a fault in it would pass every tolerance.
    """
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in qwen3_tensor_shapes(cfg).items():
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith(".bias"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif name == "model.embed_tokens.weight":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16).to(dtype)
    return out
