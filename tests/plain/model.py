"""Whole-sequence Qwen3 forward written from the reference's formulas.

One function per part, no cache, no batching tricks: every call recomputes the
full sequence.  Tensors are CPU torch tensors; the arithmetic runs in the dtype
of the weights that are passed in (float32, or float64 for tighter pins).
File:line citations point into the reference checkout (`mini_llm/...`).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- norm
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = w * (x * rsqrt(mean(x^2) + eps)) over the last dimension.

    mini_llm/nn/norm.py:42-46 (statistics in float32, weight applied after the
    cast back to the input dtype; in a float32 run both casts are no-ops).
    """
    mean_square = x.square().mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(mean_square + eps))


# --------------------------------------------------------------------------- rope
def rope_inverse_frequencies(head_dim: int, theta: float, dtype=torch.float32) -> torch.Tensor:
    """inv_freq[i] = 1 / theta^(2i/d), i = 0 .. d/2-1.  mini_llm/nn/rope.py:34-40."""
    dimensions = torch.arange(0, head_dim, 2, dtype=dtype)
    return 1.0 / (theta ** (dimensions / head_dim))


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32):
    """cos/sin of cat(angles, angles), angles[p, i] = p * inv_freq[i].

    mini_llm/nn/rope.py:74-80.  Returns two [T, d] tables.
    """
    inv = rope_inverse_frequencies(head_dim, theta, dtype)
    freqs = positions.to(dtype).unsqueeze(-1) * inv.view(1, -1)
    angles = torch.cat((freqs, freqs), dim=-1)
    return angles.cos(), angles.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """[x1, x2] -> [-x2, x1] on halves of the last dim.  mini_llm/nn/rope.py:110-114."""
    first, second = x.chunk(2, dim=-1)
    return torch.cat((-second, first), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x * cos + rotate_half(x) * sin for x [heads, T, d].  mini_llm/nn/rope.py:142-146."""
    return x * cos.unsqueeze(0) + rotate_half(x) * sin.unsqueeze(0)


# ---------------------------------------------------------------------- attention
def repeat_kv(x: torch.Tensor, repeats: int) -> torch.Tensor:
    """Each kv head serves `repeats` consecutive query heads.  mini_llm/nn/attention.py:18-33."""
    return x if repeats == 1 else x.repeat_interleave(repeats, dim=0)


def masked_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: float,
    q_positions: torch.Tensor,
    k_positions: torch.Tensor,
    window: int | None = None,
) -> torch.Tensor:
    """softmax(q k^T * scale + mask) v with mask `key_pos <= query_pos`.

    q [heads, Tq, d]; k, v [heads, Tk, d].  mini_llm/nn/attention.py:226-248
    (mask rule 231-235, scale 95-99).  `window` (not used by Qwen3) keeps only
    keys with query_pos - window < key_pos.
    """
    scores = torch.matmul(q, k.transpose(-2, -1)) * scale
    allowed = k_positions.view(1, -1) <= q_positions.view(-1, 1)
    if window is not None:
        allowed &= k_positions.view(1, -1) > (q_positions.view(-1, 1) - window)
    scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
    return torch.matmul(torch.softmax(scores, dim=-1), v)


def split_heads(x: torch.Tensor, heads: int, head_dim: int) -> torch.Tensor:
    """[T, heads*d] -> [heads, T, d]; head h owns columns h*d..(h+1)*d.  attention.py:128-132."""
    return x.view(x.shape[0], heads, head_dim).transpose(0, 1)


def qwen3_attention(
    x: torch.Tensor,
    w: dict,
    prefix: str,
    cfg: dict,
    positions: torch.Tensor,
    window: int | None = None,
    kv_override: tuple | None = None,
):
    """Projections, per-head q/k RMSNorm, RoPE, causal GQA attention, o_proj.

    mini_llm/nn/attention.py:141-254 with the Qwen3 hook 291-302.  Returns the
    block output and the (k, v) it attended to, so that a later layer may be
    told to reuse them through `kv_override`.
    """
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]

    def proj(name):
        y = x @ w[f"{prefix}.{name}.weight"].T
        bias = w.get(f"{prefix}.{name}.bias")
        return y if bias is None else y + bias

    cos, sin = rope_tables(positions, d, cfg["rope_theta"], x.dtype)
    q = split_heads(proj("q_proj"), nq, d)
    q = rms_norm(q, w[f"{prefix}.q_norm.weight"], eps)
    q = apply_rope(q, cos, sin)
    if kv_override is None:
        k = split_heads(proj("k_proj"), nkv, d)
        v = split_heads(proj("v_proj"), nkv, d)
        k = rms_norm(k, w[f"{prefix}.k_norm.weight"], eps)
        k = apply_rope(k, cos, sin)
    else:
        k, v = kv_override
    out = masked_attention(
        q, repeat_kv(k, nq // nkv), repeat_kv(v, nq // nkv),
        1.0 / math.sqrt(d), positions, positions, window,
    )
    merged = out.transpose(0, 1).reshape(x.shape[0], nq * d)
    return merged @ w[f"{prefix}.o_proj.weight"].T, (k, v)


# ---------------------------------------------------------------------------- mlp
def swiglu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)).  mini_llm/nn/mlp.py:80-87."""
    g = x @ gate.T
    return ((g * torch.sigmoid(g)) * (x @ up.T)) @ down.T


# -------------------------------------------------------------------------- model
def qwen3_layer(h, w, index, cfg, positions, window=None, kv_override=None):
    """Pre-norm residual block.  mini_llm/model/qwen.py:58-72."""
    p = f"model.layers.{index}"
    eps = cfg["rms_norm_eps"]
    attn, kv = qwen3_attention(
        rms_norm(h, w[f"{p}.input_layernorm.weight"], eps), w, f"{p}.self_attn", cfg,
        positions, window, kv_override,
    )
    h = h + attn
    x = rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
    h = h + swiglu(
        x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"]
    )
    return h, kv


def qwen3_forward(
    w: dict,
    cfg: dict,
    token_ids,
    *,
    positions=None,
    schedule=None,
    kv_from: dict | None = None,
    windows: dict | None = None,
) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.

    Embedding, layers, final norm (mini_llm/model/base.py:72-89), LM head
    (mini_llm/model/qwen.py:109-112); a tied head reuses the embedding table.
    `schedule` lists the layer indices in run order (default 0..L-1); an entry
    may repeat.  `kv_from[i] = j` makes the i-th schedule entry attend to the
    keys and values that the j-th entry produced.  `windows[layer]` gives a
    layer a sliding window.  None of the three is used by Qwen3 itself.
    """
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    dtype = w["model.embed_tokens.weight"].dtype
    if positions is None:
        positions = torch.arange(ids.shape[0])
    h = w["model.embed_tokens.weight"][ids]
    if schedule is None:
        schedule = list(range(cfg["num_hidden_layers"]))
    produced = {}
    for entry, layer in enumerate(schedule):
        source = None if kv_from is None else kv_from.get(entry)
        h, kv = qwen3_layer(
            h, w, layer, cfg, positions,
            None if windows is None else windows.get(layer),
            None if source is None else produced[source],
        )
        produced[entry] = kv
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) and "lm_head.weight" not in w else w["lm_head.weight"]
    return (h @ head.T).to(dtype)


def load_model_dir(model_dir, dtype=torch.float32):
    """Read config.json and model.safetensors of a model folder with the safetensors package."""
    from safetensors.torch import load_file

    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    weights = {k: v.to(dtype) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    return cfg, weights


# ----------------------------------------------------------------------- sampling
def filter_logits(logits: torch.Tensor, temperature: float, top_k=None, top_p: float = 1.0) -> torch.Tensor:
    """Temperature, then top-k, then nucleus filtering.  mini_llm/sampling.py:40-69."""
    z = logits.float() / temperature
    if top_k is not None and top_k < z.numel():
        kept, idx = torch.topk(z, top_k)
        z = torch.full_like(z, -torch.inf).scatter(0, idx, kept)
    if top_p < 1.0:
        s, idx = torch.sort(z, descending=True)
        p = torch.softmax(s, dim=-1)
        c = torch.cumsum(p, dim=-1)
        s = s.masked_fill(c - p >= top_p, -torch.inf)
        z = torch.empty_like(z).scatter(0, idx, s)
    return z
