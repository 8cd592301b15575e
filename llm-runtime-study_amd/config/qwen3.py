"""Typed Qwen3 dense configuration read from the keys of its config.json.

Reference: mini_llm/config.py:137-188 (fields), 226-296 (invariants), 298-354 (derived
sizes), 357-383 (Qwen3Config).  Unknown keys are ignored; `rope_scaling` and sliding-window
keys are not read, as in the reference.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Any, Mapping

from ..errors import ConfigError
from .fields import eos_token_ids, optional, read_config_json, required

DTYPE_BYTES = {"float16": 2, "bfloat16": 2, "float32": 4}


@dataclass(frozen=True)
class Qwen3Config:
    architectures: tuple[str, ...]
    model_type: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    hidden_act: str
    attention_bias: bool
    attention_dropout: float
    tie_word_embeddings: bool
    torch_dtype: str
    bos_token_id: int
    eos_token_ids: tuple[int, ...]

    ARCHITECTURE = "Qwen3ForCausalLM"
    MODEL_TYPE = "qwen3"

    @classmethod
    def from_model_dir(cls, model_dir) -> "Qwen3Config":
        return cls.from_dict(read_config_json(model_dir))

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        architectures = raw.get("architectures", [])
        if not isinstance(architectures, list) or not all(isinstance(a, str) for a in architectures):
            raise ConfigError("architectures must be a list of strings")
        if raw.get("quantization_config") is not None:
            raise ConfigError("quantized checkpoints are not supported by this runtime")
        config = cls(
            architectures=tuple(architectures),
            model_type=required(raw, "model_type", str),
            vocab_size=required(raw, "vocab_size", int),
            hidden_size=required(raw, "hidden_size", int),
            intermediate_size=required(raw, "intermediate_size", int),
            num_hidden_layers=required(raw, "num_hidden_layers", int),
            num_attention_heads=required(raw, "num_attention_heads", int),
            num_key_value_heads=required(raw, "num_key_value_heads", int),
            head_dim=required(raw, "head_dim", int),
            max_position_embeddings=required(raw, "max_position_embeddings", int),
            rms_norm_eps=float(required(raw, "rms_norm_eps", (int, float))),
            rope_theta=float(required(raw, "rope_theta", (int, float))),
            hidden_act=required(raw, "hidden_act", str),
            attention_bias=raw.get("attention_bias", False),
            attention_dropout=float(optional(raw, "attention_dropout", (int, float), 0.0)),
            tie_word_embeddings=raw.get("tie_word_embeddings", False),
            torch_dtype=required(raw, "torch_dtype", str),
            bos_token_id=required(raw, "bos_token_id", int),
            eos_token_ids=eos_token_ids(raw),
        )
        config.validate()
        return config

    def validate(self) -> None:
        if self.model_type != self.MODEL_TYPE:
            raise ConfigError(f"unsupported model_type {self.model_type!r}; expected {self.MODEL_TYPE!r}")
        if self.architectures != (self.ARCHITECTURE,):
            raise ConfigError(f"architecture must be {self.ARCHITECTURE}, got {self.architectures}")
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                "num_attention_heads must be divisible by num_key_value_heads for grouped-query attention, got "
                f"{self.num_attention_heads} and {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim must be even for rotary embeddings, got {self.head_dim}")
        if self.rms_norm_eps <= 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if self.rope_theta <= 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(f"unsupported hidden_act {self.hidden_act!r}; expected 'silu'")
        if not isinstance(self.attention_bias, bool):
            raise ConfigError("attention_bias must be boolean")
        if self.attention_dropout < 0 or self.attention_dropout >= 1:
            raise ConfigError("attention_dropout must satisfy 0 <= value < 1")
        if not isinstance(self.tie_word_embeddings, bool):
            raise ConfigError("tie_word_embeddings must be boolean")
        if self.torch_dtype not in DTYPE_BYTES:
            raise ConfigError(
                f"unsupported torch_dtype {self.torch_dtype!r}; expected one of: {', '.join(sorted(DTYPE_BYTES))}")
        for name, token in (("bos_token_id", self.bos_token_id), *(("eos_token_id", t) for t in self.eos_token_ids)):
            if not 0 <= token < self.vocab_size:
                raise ConfigError(f"{name} must be within vocabulary [0, {self.vocab_size}), got {token}")

    # ------------------------------------------------------------- derived sizes
    @property
    def query_projection_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_projection_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def queries_per_kv_head(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def validate_context_length(self, max_seq_len: int) -> None:
        if max_seq_len <= 0:
            raise ConfigError(f"max_seq_len must be positive, got {max_seq_len}")
        if max_seq_len > self.max_position_embeddings:
            raise ConfigError(f"max_seq_len {max_seq_len} exceeds the model limit {self.max_position_embeddings}")

    def kv_cache_bytes(self, max_seq_len: int, *, batch_size: int = 1, dtype: str = "bfloat16") -> int:
        """layers * 2 * batch * kv heads * positions * head_dim * bytes per scalar."""
        self.validate_context_length(max_seq_len)
        if batch_size <= 0:
            raise ConfigError(f"batch_size must be positive, got {batch_size}")
        if dtype not in DTYPE_BYTES:
            raise ConfigError(f"unsupported cache dtype {dtype!r}; expected one of: {', '.join(sorted(DTYPE_BYTES))}")
        return (self.num_hidden_layers * 2 * batch_size * self.num_key_value_heads * max_seq_len * self.head_dim
                * DTYPE_BYTES[dtype])

    def to_json_dict(self) -> dict:
        """The config.json content that reads back as this configuration."""
        raw = asdict(self)
        raw["architectures"] = list(self.architectures)
        eos = raw.pop("eos_token_ids")
        raw["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return raw
