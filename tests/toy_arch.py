"""A whole architecture that the package has never heard of, defined under tests/ and plugged in through the
registries alone: its own typed configuration (its own config.json keys), its own parts and a plain float64 forward
of the same formulas.  It is nobody's model.  Layers differ: an 'a' layer is the package's grouped-query attention
with a position encoding of the tests' own (rotary angles of squeezed positions) and a feed-forward with routing
(the likeliest of a few small experts); an 'm' layer is a mixer with state of its own (the running mean of its
inputs) and the package's SwiGLU.  A learned position table is added to the stream right after the embedding and the
logits are capped softly after the head: the two optional parts around the stack (role "transform").

Importing this module registers everything; a program of its own (the command line, bin/trace_run) imports it when
LLM_RUNTIME_STUDY_PLUGINS names it.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from llm_runtime_study_amd.config import register_architecture
from llm_runtime_study_amd.errors import ConfigError
from llm_runtime_study_amd.models import ModelSpec, ScheduleEntry
from llm_runtime_study_amd.parts import PartSpec, StateNeed, TensorSpec, register

ARCHITECTURE = "ToyMixForCausalLM"


# ------------------------------------------------------------------ configuration
@dataclass(frozen=True)
class ToyMixConfig:
    model_type: str
    vocab_size: int
    width: int
    pattern: str            # one letter a layer: 'a' attention + routed experts, 'm' running mean + SwiGLU
    heads: int
    kv_heads: int
    head_size: int
    inner: int
    experts: int
    expert_inner: int
    norm_eps: float
    rope_base: float
    rope_squeeze: float
    logit_cap: float
    max_positions: int
    eos_token_ids: tuple
    storage: str = "bfloat16"

    KEYS = ("vocab_size", "width", "pattern", "heads", "kv_heads", "head_size", "inner", "experts", "expert_inner", "norm_eps",
            "rope_base", "rope_squeeze", "logit_cap", "max_positions")

    @classmethod
    def from_dict(cls, raw: dict) -> "ToyMixConfig":
        lacking = [key for key in cls.KEYS + ("model_type", "eos_id") if key not in raw]
        if lacking:
            raise ConfigError(f"config.json lacks: {', '.join(lacking)}")
        config = cls(model_type=raw["model_type"], eos_token_ids=(int(raw["eos_id"]),), storage=raw.get("storage", "bfloat16"),
                     **{key: raw[key] for key in cls.KEYS})
        if config.model_type != "toy_mix" or not config.pattern or set(config.pattern) - set("am"):
            raise ConfigError("model_type must be 'toy_mix' and pattern a string of 'a' and 'm'")
        if config.heads % config.kv_heads or min(config.vocab_size, config.width, config.inner, config.experts) <= 0:
            raise ConfigError("sizes must be positive and heads a multiple of kv_heads")
        return config

    def validate_context_length(self, max_seq_len: int) -> None:
        if not 0 < max_seq_len <= self.max_positions:
            raise ConfigError(f"max_seq_len {max_seq_len} must be within 1..{self.max_positions}")

    def to_json_dict(self) -> dict:
        raw = {key: getattr(self, key) for key in self.KEYS}
        raw.update(architectures=[ARCHITECTURE], model_type=self.model_type, eos_id=self.eos_token_ids[0], storage=self.storage)
        return raw


# --------------------------------------------------------------------------- parts
class SqueezedRotary:
    """position: half-split rotation by the angles of position / squeeze."""

    def __init__(self, rotary_dim: int, theta: float, squeeze: float):
        self.rotary_dim, self.theta, self.squeeze = rotary_dim, theta, squeeze
        self._inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))

    def tensors(self):
        return {}

    def bind(self, weights, dtype):
        pass

    def weight_bytes(self):
        return 0

    def tables(self, ctx):
        key = ("toy_squeezed", self.rotary_dim, self.theta, self.squeeze)
        cached = ctx.memo.get(key)
        if cached is None:
            angles = (ctx.positions[:ctx.T].float() / self.squeeze)[:, None] * self._inv.to(ctx.positions.device)[None]
            cached = ctx.memo[key] = (angles.cos().contiguous(), angles.sin().contiguous())
        return cached


class LikeliestExpert:
    """feed_forward with routing: router logits in float32; the likeliest expert alone runs for a token, its output
    weighted with the router's probability: out = p_e * W2_e relu(W1_e x)."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int):
        self.h, self.i, self.e = hidden_size, intermediate_size, num_experts
        self.router = self.up = self.down = None

    def tensors(self):
        specs = {"router.weight": TensorSpec((self.e, self.h))}
        for e in range(self.e):
            specs[f"experts.{e}.up.weight"] = TensorSpec((self.i, self.h))
            specs[f"experts.{e}.down.weight"] = TensorSpec((self.h, self.i))
        return specs

    def bind(self, weights, dtype):
        self.router = weights["router.weight"].float()
        self.up = [weights[f"experts.{e}.up.weight"].to(dtype) for e in range(self.e)]
        self.down = [weights[f"experts.{e}.down.weight"].to(dtype) for e in range(self.e)]

    def weight_bytes(self):
        return 0

    def flops(self, tokens, pairs):
        return 2.0 * tokens * (self.e * self.h + 2 * self.i * self.h)       # the router, and one expert a token

    def forward(self, ctx, x, residual):
        rows = x.shape[0]
        probabilities = torch.softmax(x.float() @ self.router.T, dim=-1)
        weight, chosen = probabilities.max(dim=-1)
        for e in range(self.e):
            mine = (chosen == e).nonzero().flatten()
            if mine.numel():
                hidden = torch.relu(x[mine] @ self.up[e].T)
                residual[:rows].index_add_(0, mine, (hidden @ self.down[e].T).float() * weight[mine, None])


class RunningMean:
    """mixer with state of its own: the output at a token is W applied to the mean of all inputs of the request up to
    and including that token.  State per request: the running sum [H] and the count."""

    def __init__(self, hidden_size: int):
        self.hidden_size = hidden_size
        self.weight = None

    def tensors(self):
        return {"mix.weight": TensorSpec((self.hidden_size, self.hidden_size))}

    def bind(self, weights, dtype):
        self.weight = weights["mix.weight"].float()

    def weight_bytes(self):
        return self.weight.numel() * 4

    def cache_need(self):
        return StateNeed((self.hidden_size + 1,), torch.float32)

    def forward(self, ctx, x, residual, cache):
        start = 0
        for n, slot in zip(ctx.host_q_lens, ctx.host_slots):
            state = cache.state[slot]
            sums = state[:-1] + torch.cumsum(x[start:start + n].float(), 0)
            counts = state[-1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            residual[start:start + n] += (sums / counts[:, None]) @ self.weight.T
            state[:-1] = sums[-1]
            state[-1] = counts[-1]
            start += n


class LearnedPositions:
    """transform after the embedding: a learned row per absolute position is added to the stream."""

    def __init__(self, positions: int, hidden_size: int):
        self.positions, self.hidden_size = positions, hidden_size
        self.table = None

    def tensors(self):
        return {"weight": TensorSpec((self.positions, self.hidden_size), role="embedding")}

    def bind(self, weights, dtype):
        self.table = weights["weight"].float()

    def weight_bytes(self):
        return 0

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, h):
        h[:ctx.T] += self.table[ctx.positions[:ctx.T].long()]


class SoftCap:
    """transform after the head: logits -> cap * tanh(logits / cap)."""

    def __init__(self, cap: float):
        self.cap = cap

    def tensors(self):
        return {}

    def bind(self, weights, dtype):
        pass

    def weight_bytes(self):
        return 0

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, logits):
        logits.copy_(self.cap * torch.tanh(logits / self.cap))


NAMES_A = {"mixer": "self_attn", "feed_forward": "moe", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"}
NAMES_M = {"mixer": "mixer", "feed_forward": "mlp", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"}


def build_spec(config: ToyMixConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": config.width, "eps": config.norm_eps})
    attention = PartSpec("prenorm", {
        "mixer": PartSpec("gqa_attention", {
            "hidden_size": config.width, "num_heads": config.heads, "num_kv_heads": config.kv_heads, "head_dim": config.head_size,
            "position": PartSpec("toy_squeezed_rotary", {"rotary_dim": config.head_size, "theta": config.rope_base, "squeeze": config.rope_squeeze}),
        }),
        "feed_forward": PartSpec("toy_likeliest_expert", {"hidden_size": config.width, "intermediate_size": config.expert_inner, "num_experts": config.experts}),
        "mixer_norm": norm, "ff_norm": norm, "names": NAMES_A,
    })
    mean = PartSpec("prenorm", {
        "mixer": PartSpec("toy_running_mean", {"hidden_size": config.width}),
        "feed_forward": PartSpec("swiglu", {"hidden_size": config.width, "intermediate_size": config.inner}),
        "mixer_norm": norm, "ff_norm": norm, "names": NAMES_M,
    })
    layers = tuple(attention if letter == "a" else mean for letter in config.pattern)
    return ModelSpec(
        architecture=ARCHITECTURE, vocab_size=config.vocab_size, hidden_size=config.width, layers=layers,
        schedule=tuple(ScheduleEntry(i) for i in range(len(layers))), final_norm=norm, max_positions=config.max_positions,
        eos_token_ids=config.eos_token_ids, checkpoint_dtype=config.storage,
        after_embedding=PartSpec("toy_learned_positions", {"positions": config.max_positions, "hidden_size": config.width}),
        after_head=PartSpec("toy_soft_cap", {"cap": config.logit_cap}),
        after_embedding_prefix="model.position_table",
    )


register("position", "toy_squeezed_rotary", SqueezedRotary)
register("feed_forward", "toy_likeliest_expert", LikeliestExpert)
register("mixer", "toy_running_mean", RunningMean)
register("transform", "toy_learned_positions", LearnedPositions)
register("transform", "toy_soft_cap", SoftCap)
register_architecture(ARCHITECTURE, ToyMixConfig, build_spec)

TOY_MIX = {
    "architectures": [ARCHITECTURE], "model_type": "toy_mix", "vocab_size": 157, "width": 72, "pattern": "ama", "heads": 6, "kv_heads": 3,
    "head_size": 32, "inner": 104, "experts": 3, "expert_inner": 40, "norm_eps": 2e-5, "rope_base": 3000.0, "rope_squeeze": 2.5,
    "logit_cap": 6.0, "max_positions": 192, "eos_id": 156, "storage": "bfloat16",
}


# ------------------------------------------------------------------ the plain forward
def plain_forward(w: dict, raw: dict, ids) -> torch.Tensor:
    """Logits [T, V] of one whole sequence, every formula written out again with plain tensor operations."""
    nq, nkv, d, eps = raw["heads"], raw["kv_heads"], raw["head_size"], raw["norm_eps"]
    count = len(ids)
    positions = torch.arange(count)
    dtype = w["model.embed_tokens.weight"].dtype

    def norm(x, name):
        return w[name] * (x * torch.rsqrt(x.square().mean(-1, keepdim=True) + eps))

    def rotate(x):                      # [heads, T, d]
        inv = 1.0 / (raw["rope_base"] ** (torch.arange(0, d, 2, dtype=dtype) / d))
        angles = (positions.to(dtype) / raw["rope_squeeze"])[:, None] * inv[None]
        cos, sin = torch.cat((angles, angles), -1).cos(), torch.cat((angles, angles), -1).sin()
        first, second = x.chunk(2, -1)
        return x * cos + torch.cat((-second, first), -1) * sin

    h = w["model.embed_tokens.weight"][torch.as_tensor(ids)] + w["model.position_table.weight"][:count]
    for index, letter in enumerate(raw["pattern"]):
        p = f"model.layers.{index}"
        x = norm(h, f"{p}.input_layernorm.weight")
        if letter == "a":
            q = rotate((x @ w[f"{p}.self_attn.q_proj.weight"].T).view(count, nq, d).transpose(0, 1))
            k = rotate((x @ w[f"{p}.self_attn.k_proj.weight"].T).view(count, nkv, d).transpose(0, 1))
            v = (x @ w[f"{p}.self_attn.v_proj.weight"].T).view(count, nkv, d).transpose(0, 1)
            k, v = k.repeat_interleave(nq // nkv, 0), v.repeat_interleave(nq // nkv, 0)
            scores = q @ k.transpose(-1, -2) / math.sqrt(d)
            scores = scores.masked_fill(positions[None, :] > positions[:, None], float("-inf"))
            out = (torch.softmax(scores, -1) @ v).transpose(0, 1).reshape(count, nq * d)
            h = h + out @ w[f"{p}.self_attn.o_proj.weight"].T
            x = norm(h, f"{p}.post_attention_layernorm.weight")
            probabilities = torch.softmax(x @ w[f"{p}.moe.router.weight"].T, -1)
            weight, chosen = probabilities.max(-1)
            y = torch.zeros_like(h)
            for t in range(count):
                e = int(chosen[t])
                y[t] = weight[t] * (torch.relu(x[t] @ w[f"{p}.moe.experts.{e}.up.weight"].T) @ w[f"{p}.moe.experts.{e}.down.weight"].T)
            h = h + y
        else:
            mean = torch.cumsum(x, 0) / torch.arange(1, count + 1, dtype=dtype)[:, None]
            h = h + mean @ w[f"{p}.mixer.mix.weight"].T
            x = norm(h, f"{p}.post_attention_layernorm.weight")
            gate = x @ w[f"{p}.mlp.gate_proj.weight"].T
            h = h + ((gate * torch.sigmoid(gate)) * (x @ w[f"{p}.mlp.up_proj.weight"].T)) @ w[f"{p}.mlp.down_proj.weight"].T
    logits = norm(h, "model.norm.weight") @ w["lm_head.weight"].T
    return raw["logit_cap"] * torch.tanh(logits / raw["logit_cap"])
