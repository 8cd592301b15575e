"""Pins of the plain implementation: vectors held by the reference's own tests,
special cases that reduce to a library routine, and invariants.  Each is chosen
so that one plausible misreading (a sign, a pairing, a norm in the wrong place)
fails it.  CPU only.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from tests.plain import model as plain

from tests.helpers import random_qwen3_weights, TINY_A, TINY_B


def test_rms_norm_equation_vector():
    # reference tests/test_norm.py:11-27
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-2.0, 0.5, 1.5, 3.0]])
    w = torch.tensor([1.0, 0.5, 1.5, 2.0])
    got = plain.rms_norm(x, w, 1e-6)
    row0 = torch.tensor([1.0, 2.0, 3.0, 4.0]) / math.sqrt(7.5 + 1e-6) * w
    torch.testing.assert_close(got[0], row0)
    torch.testing.assert_close(got, F.rms_norm(x, (4,), w, 1e-6))


def test_rms_norm_eps_sits_under_the_square_root():
    """reference mini_llm/nn/norm.py:42-46: x * rsqrt(mean(x^2) + eps).  With eps = 0.5 the other readings are far
    off: x / (sqrt(mean) + eps) gives 1/1.0, eps added to the sum instead of the mean gives 1/sqrt(0.375)."""
    x = torch.tensor([[0.5, -0.5, 0.5, -0.5]])           # mean of squares 0.25
    got = plain.rms_norm(x, torch.ones(4), 0.5)
    torch.testing.assert_close(got, x / math.sqrt(0.75))
    assert not torch.allclose(got, x / (0.5 + 0.5), rtol=0.05) and not torch.allclose(got, x / math.sqrt(0.25 + 0.5 / 4), rtol=0.05)
    torch.testing.assert_close(got, F.rms_norm(x, (4,), torch.ones(4), 0.5))
    w = torch.tensor([2.0, 1.0, 0.5, 3.0])                # the weight multiplies after the normalisation
    torch.testing.assert_close(plain.rms_norm(x, w, 0.5), w * x / math.sqrt(0.75))


def test_rms_norm_half_precision_vector():
    # reference tests/test_norm.py:29-38: [300, 400] -> [0.8486, 1.1314]
    got = plain.rms_norm(torch.tensor([[300.0, 400.0]]), torch.ones(2), 1e-6)
    torch.testing.assert_close(got, torch.tensor([[0.8486, 1.1314]]), rtol=1e-3, atol=1e-3)


def test_rms_norm_invariants():
    x = torch.randn(5, 24)
    unit = plain.rms_norm(x, torch.ones(24), 1e-12)
    torch.testing.assert_close(unit.square().mean(-1), torch.ones(5))
    torch.testing.assert_close(plain.rms_norm(7.0 * x, torch.ones(24), 1e-12), unit)
    # no mean subtraction: a constant vector maps to +-1, not to 0
    torch.testing.assert_close(plain.rms_norm(torch.full((1, 8), 3.0), torch.ones(8), 1e-12), torch.ones(1, 8))


def test_qk_norm_shared_weight_vector():
    # reference tests/test_norm.py:64-85: weights 2 and 3 => k = 1.5 q
    base = torch.tensor([1.0, 2.0, 3.0, 4.0])
    q = plain.rms_norm(base.repeat(4, 3, 1), torch.full((4,), 2.0), 1e-6)
    k = plain.rms_norm(base.repeat(2, 3, 1), torch.full((4,), 3.0), 1e-6)
    torch.testing.assert_close(k[0, 0], 1.5 * q[0, 0])


def test_rope_hand_rotation_vector():
    # reference tests/test_rope.py:16-42: d=4, theta=1e4, pairs (0,2) and (1,3)
    cos, sin = plain.rope_tables(torch.tensor([0, 1]), 4, 10000.0)
    for vec in (torch.tensor([1.0, 2.0, 3.0, 4.0]), torch.tensor([-0.5, 1.5, 2.5, -3.0])):
        out = plain.apply_rope(vec.expand(1, 2, 4), cos, sin)
        torch.testing.assert_close(out[0, 0], vec)
        a, b = 1.0, 0.01
        want = torch.tensor([
            vec[0] * math.cos(a) - vec[2] * math.sin(a),
            vec[1] * math.cos(b) - vec[3] * math.sin(b),
            vec[2] * math.cos(a) + vec[0] * math.sin(a),
            vec[3] * math.cos(b) + vec[1] * math.sin(b),
        ])
        torch.testing.assert_close(out[0, 1], want)


def test_rope_invariants():
    d, theta = 16, 1e4
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)

    def dot(p, s):
        cp, sp = plain.rope_tables(torch.tensor([p]), d, theta, torch.float64)
        cs, ss = plain.rope_tables(torch.tensor([s]), d, theta, torch.float64)
        return (plain.apply_rope(q, cp, sp) * plain.apply_rope(k, cs, ss)).sum()

    # only distances count
    torch.testing.assert_close(dot(9, 4), dot(105, 100))
    assert abs(dot(9, 4) - dot(9, 5)) > 1e-6
    # norm preserving (reference tests/test_rope.py:44-58)
    c, s = plain.rope_tables(torch.arange(7), d, theta, torch.float64)
    x = torch.randn(3, 7, d, dtype=torch.float64)
    torch.testing.assert_close(plain.apply_rope(x, c, s).norm(dim=-1), x.norm(dim=-1))
    # inverse frequencies: first is 1, last is theta^-(d-2)/d
    inv = plain.rope_inverse_frequencies(d, theta, torch.float64)
    assert inv[0] == 1.0 and abs(inv[-1] - theta ** (-(d - 2) / d)) < 1e-15


def test_attention_reduces_to_library():
    heads, t, d = 3, 9, 8
    q, k, v = (torch.randn(heads, t, d) for _ in range(3))
    pos = torch.arange(t)
    got = plain.masked_attention(q, k, v, 1 / math.sqrt(d), pos, pos)
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    # no mask at all: every query sits after every key
    got = plain.masked_attention(q, k, v, 0.3, torch.full((t,), 100), pos)
    want = torch.softmax(q @ k.transpose(-1, -2) * 0.3, -1) @ v
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_attention_special_cases():
    d = 4
    q = torch.randn(2, 1, d)
    v = torch.randn(2, 5, d)
    # one key => output is its value
    out = plain.masked_attention(q, torch.randn(2, 1, d), v[:, :1], 0.5, torch.tensor([0]), torch.tensor([0]))
    torch.testing.assert_close(out, v[:, :1])
    # identical keys => mean of the values
    k = torch.randn(2, 1, d).expand(2, 5, d)
    out = plain.masked_attention(q, k, v, 0.5, torch.tensor([4]), torch.arange(5))
    torch.testing.assert_close(out, v.mean(1, keepdim=True), rtol=1e-5, atol=1e-6)
    # window 2 at position 4 sees keys 3 and 4 only
    out = plain.masked_attention(q, k, v, 0.5, torch.tensor([4]), torch.arange(5), window=2)
    torch.testing.assert_close(out, v[:, 3:].mean(1, keepdim=True), rtol=1e-5, atol=1e-6)


def test_gqa_head_map():
    # reference tests/test_attention.py:88-96: kv heads [1, 2] serve query heads [1, 1, 2, 2]
    states = torch.tensor([[[1.0]], [[2.0]]])
    torch.testing.assert_close(plain.repeat_kv(states, 2)[:, 0, 0], torch.tensor([1.0, 1.0, 2.0, 2.0]))


def test_qwen3_attention_matches_manual_reference():
    # the recipe of reference tests/test_attention.py:47-84 with unit norm weights and all tokens at one
    # position: pins projections, head split, grouping, scale and the output projection; the order of norm
    # and rotation and the mask are pinned by the next test
    torch.manual_seed(11)
    cfg = dict(num_attention_heads=2, num_key_value_heads=1, head_dim=2, rms_norm_eps=1e-6, rope_theta=1e4)
    w = {
        "a.q_proj.weight": torch.randn(4, 2), "a.k_proj.weight": torch.randn(2, 2),
        "a.v_proj.weight": torch.randn(2, 2), "a.o_proj.weight": torch.randn(2, 4),
        "a.q_norm.weight": torch.ones(2), "a.k_norm.weight": torch.ones(2),
    }
    x = torch.tensor([[1.0, 2.0], [-1.0, 0.5], [0.25, -0.75]])
    # all positions equal => rotation cancels in q.k, so the no-rope manual recipe applies
    got, _ = plain.qwen3_attention(x, w, "a", cfg, torch.zeros(3, dtype=torch.long))
    q = (x @ w["a.q_proj.weight"].T).view(3, 2, 2).transpose(0, 1)
    k = (x @ w["a.k_proj.weight"].T).view(3, 1, 2).transpose(0, 1)
    v = (x @ w["a.v_proj.weight"].T).view(3, 1, 2).transpose(0, 1)
    q = q * torch.rsqrt(q.square().mean(-1, keepdim=True) + 1e-6)
    k = k * torch.rsqrt(k.square().mean(-1, keepdim=True) + 1e-6)
    s = (q @ k.repeat_interleave(2, 0).transpose(-1, -2)) / math.sqrt(2)
    # equal positions: the mask key_pos <= query_pos lets every key through
    o = torch.softmax(s, -1) @ v.repeat_interleave(2, 0)
    want = o.transpose(0, 1).reshape(3, 4) @ w["a.o_proj.weight"].T
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_qwen3_attention_normalises_before_it_rotates_and_masks_later_keys():
    """Heads of two dims are one rotary pair, so the rotation is a plain 2-D rotation by the position (theta plays
    no part).  With norm weights (2, 0.5) rotating before normalising gives other numbers, and with positions
    0, 1, 2 a key after the query must not count (reference mini_llm/nn/attention.py:231-248, 286-302)."""
    torch.manual_seed(12)
    cfg = dict(num_attention_heads=2, num_key_value_heads=1, head_dim=2, rms_norm_eps=1e-6, rope_theta=1e4)
    w = {
        "a.q_proj.weight": torch.randn(4, 2), "a.k_proj.weight": torch.randn(2, 2),
        "a.v_proj.weight": torch.randn(2, 2), "a.o_proj.weight": torch.randn(2, 4),
        "a.q_norm.weight": torch.tensor([2.0, 0.5]), "a.k_norm.weight": torch.tensor([0.25, 3.0]),
    }
    x = torch.tensor([[1.0, 2.0], [-1.0, 0.5], [0.25, -0.75]])
    positions = torch.tensor([0, 1, 2])
    got, _ = plain.qwen3_attention(x, w, "a", cfg, positions)

    def rotate(t, swap_order=False):          # t [heads, tokens, 2]
        c, s_ = torch.cos(positions.float()), torch.sin(positions.float())
        return torch.stack((t[..., 0] * c - t[..., 1] * s_, t[..., 1] * c + t[..., 0] * s_), -1)

    def norm(t, weight):
        return t * torch.rsqrt(t.square().mean(-1, keepdim=True) + 1e-6) * weight

    def recipe(norm_first: bool, causal: bool):
        q = (x @ w["a.q_proj.weight"].T).view(3, 2, 2).transpose(0, 1)
        k = (x @ w["a.k_proj.weight"].T).view(3, 1, 2).transpose(0, 1)
        v = (x @ w["a.v_proj.weight"].T).view(3, 1, 2).transpose(0, 1)
        if norm_first:
            q, k = rotate(norm(q, w["a.q_norm.weight"])), rotate(norm(k, w["a.k_norm.weight"]))
        else:
            q, k = norm(rotate(q), w["a.q_norm.weight"]), norm(rotate(k), w["a.k_norm.weight"])
        scores = (q @ k.repeat_interleave(2, 0).transpose(-1, -2)) / math.sqrt(2)
        if causal:
            scores = scores.masked_fill(torch.triu(torch.ones(3, 3, dtype=torch.bool), 1), -torch.inf)
        o = torch.softmax(scores, -1) @ v.repeat_interleave(2, 0)
        return o.transpose(0, 1).reshape(3, 4) @ w["a.o_proj.weight"].T

    torch.testing.assert_close(got, recipe(True, True), rtol=1e-5, atol=1e-6)
    assert not torch.allclose(got, recipe(False, True), rtol=1e-2, atol=1e-3)      # norm after the rotation: other numbers
    assert not torch.allclose(got, recipe(True, False), rtol=1e-2, atol=1e-3)      # no mask: other numbers


def test_swiglu_vector():
    # reference tests/test_mlp.py:12-30
    x = torch.tensor([[1.0, -2.0], [0.5, 3.0]])
    g = torch.tensor([[1.0, 0.5], [-0.5, 2.0], [1.5, -1.0]])
    u = torch.tensor([[0.25, 1.0], [2.0, -0.5], [-1.0, 0.75]])
    dn = torch.tensor([[1.0, -0.5, 0.25], [-0.25, 0.75, 1.5]])
    want = F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), dn)
    torch.testing.assert_close(plain.swiglu(x, g, u, dn), want)
    torch.testing.assert_close(plain.swiglu(x, g, torch.zeros_like(u), dn), torch.zeros(2, 2))


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_model_invariants(cfg):
    w = random_qwen3_weights(cfg, seed=3, dtype=torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (13,))
    logits = plain.qwen3_forward(w, cfg, ids)
    assert logits.shape == (13, cfg["vocab_size"])
    # causality: changing token j leaves logits before j untouched
    ids2 = ids.clone()
    ids2[8] = (ids2[8] + 1) % cfg["vocab_size"]
    logits2 = plain.qwen3_forward(w, cfg, ids2)
    torch.testing.assert_close(logits2[:8], logits[:8], rtol=0, atol=0)
    assert not torch.allclose(logits2[8:], logits[8:])
    # only distances count: shifting all positions changes nothing
    shifted = plain.qwen3_forward(w, cfg, ids, positions=torch.arange(13) + 29)
    torch.testing.assert_close(shifted, logits, rtol=1e-9, atol=1e-9)
    # zeroed o_proj and down_proj => logits = head(norm(embed))
    wz = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        wz[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
        wz[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.mlp.down_proj.weight"])
    head = wz.get("lm_head.weight", wz["model.embed_tokens.weight"])
    want = plain.rms_norm(wz["model.embed_tokens.weight"][ids], wz["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    torch.testing.assert_close(plain.qwen3_forward(wz, cfg, ids), want)


def _one_token_by_hand(w, cfg, token, eps, parallel=False, embedding_scale=1.0):
    """Logits of a sequence of one token, written with library routines only.  One token attends to itself with
    weight 1, so attention is o_proj of its own value heads, each repeated for the query heads of its group: no
    rotation, no q or k, no softmax.  mini_llm/model/qwen.py:58-72 (the block), mini_llm/model/base.py:72-89 (embedding
    without a multiplier for this family, final norm), mini_llm/model/qwen.py:109-112 (head)."""
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    h = embedding_scale * w["model.embed_tokens.weight"][token]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        x = F.rms_norm(h, h.shape, w[f"{p}.input_layernorm.weight"], eps)
        v = F.linear(x, w[f"{p}.self_attn.v_proj.weight"], w.get(f"{p}.self_attn.v_proj.bias"))
        merged = v.view(nkv, 1, d).expand(nkv, nq // nkv, d).reshape(nq * d)
        attn = F.linear(merged, w[f"{p}.self_attn.o_proj.weight"])
        after = h + attn
        y = F.rms_norm(h if parallel else after, h.shape, w[f"{p}.post_attention_layernorm.weight"], eps)
        mlp = F.linear(F.silu(F.linear(y, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(y, w[f"{p}.mlp.up_proj.weight"]), w[f"{p}.mlp.down_proj.weight"])
        h = after + mlp
    head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
    return F.linear(F.rms_norm(h, h.shape, w["model.norm.weight"], eps), head)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_one_token_reduces_to_library_routines_and_tells_the_block_readings_apart(cfg):
    """The block is sequential (the feed-forward reads the norm of the stream the attention has already been added
    to: the composition the reference's own test states, tests/test_qwen_model.py:93-111) and the embedding enters
    the stream unscaled.  A block whose feed-forward read the norm of the layer's input (both branches side by side),
    or an embedding scaled by sqrt(hidden), gives other logits by far: the norms cancel a scale inside the branches,
    but not in the sum with their output."""
    w = random_qwen3_weights(cfg, seed=6, dtype=torch.float64)
    eps = cfg["rms_norm_eps"]
    for token in (0, 5, cfg["vocab_size"] - 1):
        got = plain.qwen3_forward(w, cfg, [token])[0]
        torch.testing.assert_close(got, _one_token_by_hand(w, cfg, token, eps), rtol=1e-9, atol=1e-9)
        side_by_side = _one_token_by_hand(w, cfg, token, eps, parallel=True)
        scaled = _one_token_by_hand(w, cfg, token, eps, embedding_scale=cfg["hidden_size"] ** 0.5)
        assert (got - side_by_side).norm() > 0.05 * got.norm() and (got - scaled).norm() > 0.05 * got.norm()


def test_q_and_k_norms_use_the_models_eps():
    """mini_llm/model/qwen.py:33,44-47: the per-head norms of q and k take rms_norm_eps like the other norms.  With
    eps 0.3 a reading that hard-codes 1e-6 there is far off.  Two tokens: heads normalised by the library's rms_norm,
    rotated (pinned above), attended by the library's causal attention."""
    cfg = dict(TINY_A, rms_norm_eps=0.3, num_hidden_layers=1)
    w = random_qwen3_weights(cfg, seed=8, dtype=torch.float64)
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    x = torch.randn(2, cfg["hidden_size"], dtype=torch.float64)
    got, _ = plain.qwen3_attention(x, w, "model.layers.0.self_attn", cfg, torch.arange(2))

    def by_hand(eps):
        p = "model.layers.0.self_attn"
        q = F.rms_norm((x @ w[f"{p}.q_proj.weight"].T).view(2, nq, d), (d,), w[f"{p}.q_norm.weight"], eps)
        k = F.rms_norm((x @ w[f"{p}.k_proj.weight"].T).view(2, nkv, d), (d,), w[f"{p}.k_norm.weight"], eps)
        v = (x @ w[f"{p}.v_proj.weight"].T).view(2, nkv, d)
        cos, sin = plain.rope_tables(torch.arange(2), d, cfg["rope_theta"], x.dtype)
        q, k = plain.apply_rope(q.transpose(0, 1), cos, sin), plain.apply_rope(k.transpose(0, 1), cos, sin)
        k, v = k.repeat_interleave(nq // nkv, 0), v.transpose(0, 1).repeat_interleave(nq // nkv, 0)
        out = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
        return out.transpose(0, 1).reshape(2, nq * d) @ w[f"{p}.o_proj.weight"].T

    torch.testing.assert_close(got, by_hand(0.3), rtol=1e-9, atol=1e-9)
    assert (got[1] - by_hand(1e-6)[1]).norm() > 0.02 * got[1].norm()


def test_tied_head_uses_embedding():
    w = random_qwen3_weights(TINY_A, seed=1, dtype=torch.float64)
    assert "lm_head.weight" not in w
    untied = dict(w)
    untied["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    cfg2 = dict(TINY_A, tie_word_embeddings=False)
    ids = [3, 9, 200, 17]
    torch.testing.assert_close(plain.qwen3_forward(w, TINY_A, ids), plain.qwen3_forward(untied, cfg2, ids))


def test_filter_logits_vectors():
    # reference tests/test_generation.py top-p: probs .60 .25 .10 .05, p=.70 keeps two
    logits = torch.log(torch.tensor([0.60, 0.25, 0.10, 0.05]))
    kept = plain.filter_logits(logits, 1.0, None, 0.70)
    assert torch.isfinite(kept).tolist() == [True, True, False, False]
    kept = plain.filter_logits(torch.tensor([1.0, 4.0, 2.0, 3.0]), 2.0, 2, 1.0)
    assert torch.isfinite(kept).tolist() == [False, True, False, True]
    torch.testing.assert_close(kept[1], torch.tensor(2.0))
