"""Qwen3 dense: configuration -> ModelSpec.

Reference mini_llm/model/qwen.py:18-112: every layer is a pre-norm block of grouped-query
attention with per-head q/k RMSNorm (same eps as the other norms, qwen.py:33,44-47) and rotary
positions, and a SwiGLU feed-forward; all layers attend to the full context; checkpoint
names are the reference's module paths (mini_llm/checkpoint.py:287-344).  The dense reference
always stores lm_head.weight; here a tied configuration may omit it and reuse the embedding.
"""

from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..parts import PartSpec
from .spec import ModelSpec, ScheduleEntry

LAYER_NAMES = {"mixer": "self_attn", "feed_forward": "mlp", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"}


def build_spec(config: Qwen3Config) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": config.hidden_size, "eps": config.rms_norm_eps})
    block = PartSpec("prenorm", {
        "mixer": PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size,
            "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "position": PartSpec("rope_half", {"rotary_dim": config.head_dim, "theta": config.rope_theta}),
            "qk_norm": True,
            "qk_norm_eps": config.rms_norm_eps,
            "bias": config.attention_bias,
        }),
        "feed_forward": PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}),
        "mixer_norm": norm,
        "ff_norm": norm,
        "names": LAYER_NAMES,
    })
    return ModelSpec(
        architecture=Qwen3Config.ARCHITECTURE,
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        layers=tuple(block for _ in range(config.num_hidden_layers)),
        schedule=tuple(ScheduleEntry(i) for i in range(config.num_hidden_layers)),
        final_norm=norm,
        max_positions=config.max_position_embeddings,
        eos_token_ids=config.eos_token_ids,
        bos_token_id=config.bos_token_id,
        tie_head=config.tie_word_embeddings,
        checkpoint_dtype=config.torch_dtype,
    )
