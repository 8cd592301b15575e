"""Parts that the framework has never heard of, defined here and plugged in through the registry:
a position encoding (rotary angles of interpolated positions) and a feed-forward with routing
(top-1 of a few small experts), in one layer of a model whose other layer is built from the
package's own parts.  Nothing under the package changes; the model is stepped in portions, single
tokens and mixed batches and compared with a plain composition of the same formulas."""

import math

import numpy as np
import pytest
import torch

from tests.plain import model as plain
from tests.test_parts_gpu import DTYPES, build_runner, close

pytestmark = pytest.mark.gpu


class InterpolatedRotary:
    """Half-split rotation by the angles of position / factor (positions squeezed into a shorter
    range).  Tables are made with library calls on the device, once per step."""

    def __init__(self, rotary_dim: int, theta: float, factor: float):
        self.rotary_dim, self.theta, self.factor = rotary_dim, theta, factor
        self._inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))

    def tensors(self):
        return {}

    def bind(self, weights, dtype):
        pass

    def weight_bytes(self):
        return 0

    def tables(self, ctx):
        key = ("toy_interpolated", self.rotary_dim, self.theta, self.factor)
        cached = ctx.memo.get(key)
        if cached is None:
            angles = (ctx.positions[:ctx.T].float() / self.factor)[:, None] * self._inv.to(ctx.positions.device)[None]
            cached = ctx.memo[key] = (angles.cos().contiguous(), angles.sin().contiguous())
        return cached


class TopOneExperts:
    """Feed-forward with routing: router logits in float32, the most likely expert alone runs for a
    token, its output weighted with the router's probability.  out = p_e * W2_e relu(W1_e x)."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int):
        from llm_runtime_study_amd.parts import TensorSpec
        self.h, self.i, self.e = hidden_size, intermediate_size, num_experts
        self._specs = {"router.weight": TensorSpec((num_experts, hidden_size))}
        for e in range(num_experts):
            self._specs[f"experts.{e}.up.weight"] = TensorSpec((intermediate_size, hidden_size))
            self._specs[f"experts.{e}.down.weight"] = TensorSpec((hidden_size, intermediate_size))
        self.router = self.up = self.down = None

    def tensors(self):
        return dict(self._specs)

    def bind(self, weights, dtype):
        self.router = weights["router.weight"].float()
        self.up = [weights[f"experts.{e}.up.weight"].to(dtype) for e in range(self.e)]
        self.down = [weights[f"experts.{e}.down.weight"].to(dtype) for e in range(self.e)]

    def weight_bytes(self):
        return 0

    routes = []          # the expert of every row of every call, for the test to read

    def forward(self, ctx, x, residual):
        rows = x.shape[0]
        probabilities = torch.softmax(x.float() @ self.router.T, dim=-1)
        weight, chosen = probabilities.max(dim=-1)
        TopOneExperts.routes.append(chosen.cpu())
        for e in range(self.e):
            mine = (chosen == e).nonzero().flatten()
            if mine.numel():
                hidden = torch.relu(x[mine] @ self.up[e].T)
                residual[:rows].index_add_(0, mine, (hidden @ self.down[e].T).float() * weight[mine, None])


def plain_toy_model(w, cfg, ids, forced=None):
    """Layer 0: attention with interpolated rotary positions, then top-1 experts.  Layer 1: the
    Qwen3 block.  Float64 throughout.  `forced`: experts to use instead of the most likely ones.
    Also returns the experts used and, per token, how far the most likely expert leads the second."""
    nq, nkv, d, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    positions = torch.arange(len(ids))
    h = w["model.embed_tokens.weight"][torch.as_tensor(ids)]
    p = "model.layers.0"
    x = plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
    cos, sin = plain.rope_tables(positions.double() / cfg["factor"], d, cfg["rope_theta"], torch.float64)
    q = plain.apply_rope(plain.rms_norm(plain.split_heads(x @ w[f"{p}.self_attn.q_proj.weight"].T, nq, d), w[f"{p}.self_attn.q_norm.weight"], eps), cos, sin)
    k = plain.apply_rope(plain.rms_norm(plain.split_heads(x @ w[f"{p}.self_attn.k_proj.weight"].T, nkv, d), w[f"{p}.self_attn.k_norm.weight"], eps), cos, sin)
    v = plain.split_heads(x @ w[f"{p}.self_attn.v_proj.weight"].T, nkv, d)
    out = plain.masked_attention(q, plain.repeat_kv(k, nq // nkv), plain.repeat_kv(v, nq // nkv), 1 / math.sqrt(d), positions, positions)
    h = h + out.transpose(0, 1).reshape(len(ids), nq * d) @ w[f"{p}.self_attn.o_proj.weight"].T
    x = plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
    probabilities = torch.softmax(x @ w[f"{p}.moe.router.weight"].T, dim=-1)
    top = probabilities.topk(2, dim=-1)
    chosen = top.indices[:, 0] if forced is None else forced
    lead = top.values[:, 0] - top.values[:, 1]
    y = torch.zeros_like(h)
    for t in range(len(ids)):
        e = int(chosen[t])
        y[t] = probabilities[t, e] * (torch.relu(x[t] @ w[f"{p}.moe.experts.{e}.up.weight"].T) @ w[f"{p}.moe.experts.{e}.down.weight"].T)
    h = h + y
    h, _ = plain.qwen3_layer(h, w, 1, cfg, positions)
    return plain.rms_norm(h, w["model.norm.weight"], eps) @ w["lm_head.weight"].T, chosen, lead


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_position_encoding_and_routed_feed_forward_beside_the_packages_own_parts(dtype):
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.models import DecoderModel, ModelSpec, ScheduleEntry
    from llm_runtime_study_amd.parts import PartSpec, register
    from llm_runtime_study_amd.weights import random_tensors

    register("position", "toy_interpolated_rotary", InterpolatedRotary)
    register("feed_forward", "toy_top_one_experts", TopOneExperts)
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32, "rms_norm_eps": 1e-5, "rope_theta": 5000.0, "factor": 4.0}
    hidden, vocab, inter, experts = 80, 131, 112, 3
    nq, nkv, d, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})

    def attention(position):
        return PartSpec("gqa_attention", {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
                                          "position": position, "qk_norm": True, "qk_norm_eps": eps})

    toy_layer = PartSpec("prenorm", {
        "mixer": attention(PartSpec("toy_interpolated_rotary", {"rotary_dim": d, "theta": cfg["rope_theta"], "factor": cfg["factor"]})),
        "feed_forward": PartSpec("toy_top_one_experts", {"hidden_size": hidden, "intermediate_size": 48, "num_experts": experts}),
        "mixer_norm": norm, "ff_norm": norm,
        "names": {"mixer": "self_attn", "feed_forward": "moe", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"},
    })
    own_layer = PartSpec("prenorm", {
        "mixer": attention(PartSpec("rope_half", {"rotary_dim": d, "theta": cfg["rope_theta"]})),
        "feed_forward": PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter}),
        "mixer_norm": norm, "ff_norm": norm,
        "names": {"mixer": "self_attn", "feed_forward": "mlp", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"},
    })
    spec = ModelSpec(architecture="ToyRoutedInterpolated", vocab_size=vocab, hidden_size=hidden, layers=(toy_layer, own_layer),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm, max_positions=512)
    weights = random_tensors(DecoderModel(spec).tensors(), 11, torch.bfloat16, "scaled")
    weights["model.layers.0.moe.router.weight"] = weights["model.layers.0.moe.router.weight"] * 4      # clearer decisions
    runner = build_runner(spec, weights, dtype)
    assert not runner.use_graph                      # parts of unknown make run eagerly
    # equal attention needs share one group of pages although their position encodings differ
    assert [g.entries for g in runner.cache.groups] == [[0, 1]]
    rng = np.random.default_rng(4)
    requests = {key: rng.integers(0, vocab, n).tolist() for key, n in (("a", 70), ("b", 33), ("c", 45))}
    double = {k: v.double() for k, v in weights.items()}
    TopOneExperts.routes = []
    plan = [{"a": 40}, {"a": 1, "b": 20}, {"a": 2, "b": 1}, {"a": 27, "b": 12, "c": 3}, {"c": 40}, {"c": 1}, {"c": 1}]
    caches, progress, got = {}, {key: 0 for key in requests}, {key: [] for key in requests}
    for step in plan:
        entries = []
        for key, n in step.items():
            if key not in caches:
                caches[key] = runner.cache.admit(key)
            at = progress[key]
            entries.append(StepEntry(caches[key], requests[key][at:at + n], list(range(n))))
            progress[key] = at + n
        logits = runner.step(entries)
        row = 0
        for key, n in step.items():
            got[key].append(logits[row:row + n].clone())
            row += n
            if progress[key] == len(requests[key]):
                runner.cache.release(caches[key])
    assert all(progress[key] == len(ids) for key, ids in requests.items())
    # the experts the engine used, per request and position (one call of the toy part per step)
    used = {key: [] for key in requests}
    for step, chosen in zip(plan, TopOneExperts.routes):
        row = 0
        for key, n in step.items():
            used[key].append(chosen[row:row + n])
            row += n
    seen = set()
    for key, ids in requests.items():
        engine_routes = torch.cat(used[key])
        _, own, lead = plain_toy_model(double, cfg, ids)
        differ = engine_routes != own
        if dtype == torch.float32:
            assert not differ.any()
        else:
            # rounding to bfloat16 may turn a near-tie of two experts; then the plain model follows
            # the engine's choice, and the tie must have been a near one
            assert (lead[differ] < 0.05).all() and differ.float().mean() < 0.1
        seen.update(engine_routes.tolist())
        want, _, _ = plain_toy_model(double, cfg, ids, forced=engine_routes)
        close(torch.cat(got[key]), want, dtype, f32=1e-4)
    assert seen == set(range(experts))               # every expert had tokens
    runner.cache.check_invariants()
