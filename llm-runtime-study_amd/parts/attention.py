"""Grouped-query causal attention over the paged cache.

Reference mini_llm/nn/attention.py:141-254: q/k/v projections of the normed input, head
split (head h owns columns h*d..(h+1)*d), optional per-head RMSNorm of q and k over head_dim
with one weight for all q heads and one for all k heads (Qwen3, 291-302), rotation of q and k
by the token's absolute position, write of k and v into the cache, softmax(q k^T * scale) v
over cached positions j <= p (mask rule 231-235; scale 1/sqrt(d) unless given, 95-99), kv head
h // (nq/nkv) for query head h (18-33), then the output projection without bias.

q, k and v come from one stacked [nq*d + 2*nkv*d, H] product.  When `kv_shared` is set the
layer owns no keys or values: it projects queries only and attends to the cache of the layer
it is told to read.  `window` keeps keys with p - window < j <= p.
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PagedKVNeed, Part, PartSpec, TensorSpec, create, length_class, register
from .linear import ScaledRows, kernels_of, linear, materialize, rows_of, workspace_of


class GQAAttention(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True   # ... and nothing but this package's kernels, with arguments that follow the step's shape alone
    takes_lazy_norm = True
    begins_next_norm = True
    wants_query_groups = True   # ragged steps go to a kernel that walks groups of a request's consecutive tokens

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, *,
                 position: PartSpec = PartSpec("none"), qk_norm: bool = False, qk_norm_eps: float = 1e-6,
                 bias: bool = False, scale: float | None = None, window: int | None = None,
                 kv_shared: bool = False):
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads), ("head_dim", head_dim)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads must be divisible by num_kv_heads, got {num_heads} and {num_kv_heads}")
        if scale is not None and (not math.isfinite(scale) or scale <= 0):
            raise ValueError(f"scale must be finite and positive, got {scale}")
        if window is not None and window <= 0:
            raise ValueError(f"window must be positive when given, got {window}")
        if qk_norm and qk_norm_eps <= 0:
            raise ValueError(f"qk_norm_eps must be positive, got {qk_norm_eps}")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.position = create("position", position)
        self.qk_norm, self.qk_norm_eps, self.bias = qk_norm, qk_norm_eps, bias
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
        self.window, self.kv_shared = window, kv_shared
        self.w_qkv = self.b_qkv = self.w_o = self.q_norm = self.k_norm = None

    # ------------------------------------------------------------------ weights
    def tensors(self):
        h, d = self.hidden_size, self.head_dim
        names = ("q_proj",) if self.kv_shared else ("q_proj", "k_proj", "v_proj")
        widths = {"q_proj": self.num_heads * d, "k_proj": self.num_kv_heads * d, "v_proj": self.num_kv_heads * d}
        specs = {f"{n}.weight": TensorSpec((widths[n], h)) for n in names}
        if self.bias:
            specs.update({f"{n}.bias": TensorSpec((widths[n],), role="bias") for n in names})
        specs["o_proj.weight"] = TensorSpec((h, self.num_heads * d))
        if self.qk_norm:
            specs["q_norm.weight"] = TensorSpec((d,), role="norm")
            if not self.kv_shared:
                specs["k_norm.weight"] = TensorSpec((d,), role="norm")
        return specs

    def bind(self, weights, dtype):
        names = ("q_proj",) if self.kv_shared else ("q_proj", "k_proj", "v_proj")
        self.w_qkv = torch.cat([weights[f"{n}.weight"] for n in names], 0).to(dtype).contiguous()
        self.b_qkv = torch.cat([weights[f"{n}.bias"] for n in names], 0).to(dtype).contiguous() if self.bias else None
        self.w_o = weights["o_proj.weight"].to(dtype).contiguous()
        if self.qk_norm:
            self.q_norm = weights["q_norm.weight"]
            self.k_norm = weights["k_norm.weight"] if not self.kv_shared else self.q_norm

    def weight_bytes(self):
        return (self.w_qkv.numel() + self.w_o.numel()) * self.w_o.element_size()

    def flops(self, tokens, pairs):
        if self.window is not None:
            pairs = min(pairs, tokens * self.window)
        # the projections, then scores and weighted values: two products of head_dim per pair and query head
        return super().flops(tokens, pairs) + 4.0 * pairs * self.num_heads * self.head_dim

    def cache_need(self):
        if self.kv_shared:
            return None
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    @staticmethod
    def _decode_splits(workgroups: int, longest: int, bound: int, page_size: int) -> int:
        """Into how many workgroups the keys of one decode token are divided: enough to give every
        compute unit two when the batch alone does not (measured on MI355X inside the 8-request
        decode step at 2,048 tokens of context: 8 splits 4.58 ms, 4 splits 4.61 ms), but at least
        256 keys each (a power of two that follows the length's class, not the length); and enough
        that the block table entries of one workgroup (at most 4,096) fit its LDS for contexts up
        to `bound`."""
        units = ops.compute_units()
        # from five workgroups for every eight units on, the batch alone does as well or better, and there is nothing
        # to merge (2,048 tokens of context, batch 20 / 24 / 32: 37.8 / 42.0 / 52.7 us undivided against 40.1 / 45 /
        # 54.4 us with the 4 / 3 / 2 parts that two workgroups a unit would ask for; the same at 8,192 tokens)
        wanted = 1 if 8 * workgroups >= 5 * units else -(-2 * units // workgroups)
        # between one and one and a half workgroups a unit some units have two where the others have one, and with
        # contexts of 2,048 tokens and more the second round costs more than a merge: two parts (40 query heads on 8:
        # batch 33 / 40 / 44 / 48 at 2,048 tokens 72.6 / 75.1 / 77.9 / 79.7 us undivided, 66.5 / 71.5 / 73.3 / 78.2 in two parts;
        # at 4,096 tokens 140 / 144 / 148 / 151 against 122 / 129 / 134 / 144; at 1,024 tokens and from batch 52 on nothing
        # is gained; four parts are better still up to batch 40 and worse from 44 on, and a graph serves both)
        if units < workgroups <= units + units // 2 and length_class(longest) >= 2048:
            wanted = 2
        return max(1, min(wanted, length_class(longest) // 256, 64), -(-bound // (4096 * page_size)))

    @staticmethod
    def _prefill_splits(workgroups: int, longest: int, outputs: int, heads_per_group: int = 4, tokens: int = 0) -> int:
        """Into how many workgroups the keys of every query group of a ragged step are divided: one, unless
        the groups alone leave compute units idle (a last portion of a prompt, a short portion after a long
        context), and never from two workgroups a unit on.  Partial results (float32, `outputs` values per split)
        stay within 256 MB.  Measured on
        MI355X, 32 query heads on 8 kv heads:
          * contexts of 16,384 tokens and more: towards eight workgroups a unit, at least 1,024 keys each
            (32,768 tokens of context: 1 token 1,161 -> 57 us with 32 splits, 64 tokens 1,165 -> 105 us with
            16, 512 tokens 1,186 -> 576 us with 8);
          * shorter contexts: towards two workgroups a unit, at least 256 keys each (2,048 tokens of context: 64 tokens 42.5 -> 18.6 us with 8 splits, 256 tokens 43.2 -> 32.4 with
            4, 512 tokens 87.5 -> 76.4 with 2, but 1,024 tokens 96.8 -> 127 and 2,032 tokens 111 -> 173 with 2:
            what the merge reads and writes grows with the tokens, what a split saves with the context).  So under
            16,384 tokens of context the keys are divided only where the longest context is at least four times the
            step's `tokens` (undivided against 2 splits with their merge: 512 tokens after 0 / 512 / 1,024 / 1,536:
            16.9 / 26.6 / 36.2 / 45.8 against 24.4 / 30.5 / 36.9 / 42.9 us; 256 tokens after 256 / 512 / 768 / 1,024:
            16.5 / 21.1 / 25.7 / 30.2 against 18.8 / 20.3 / 23.1 / 25.6 us; 128 tokens after 0 / 256 / 512: 14.4 / 14.1 /
            18.5 against 16.2 / 16.8 / 17.1 us).
        A kv group of five to eight heads walks the keys once with a wave for every head while the launch is at
        most two workgroups a unit; that walk is short enough that one workgroup a unit is the aim (40 heads on
        8: 512 tokens after 1,536 54 us undivided against 72 with 2; 256 tokens 51 -> 43 with 2, 128 tokens
        after 8,064 177 -> 59 with 4, 64 tokens after 2,000 50 -> 22 with 8); from 16,384 tokens of context on the rule
        for long contexts holds for them too (512 tokens after 32,256: 697 us undivided, 617 with 8)."""
        units = ops.compute_units()
        within = (64 << 20) // max(outputs, 1)
        if workgroups >= 2 * units:      # (2,048 tokens in groups of 32 after 30,720: 1,071 us undivided, 1,115 with 2)
            return 1
        if longest < 16384 and longest < 4 * tokens:
            return 1
        if heads_per_group > 4 and workgroups <= units and longest < 16384:
            return max(1, min(-(-units // workgroups), longest // 256, 32, within))
        if longest >= 16384:
            return max(1, min(-(-8 * units // workgroups), longest // 1024, 32, within))
        return max(1, min(-(-2 * units // workgroups), longest // 256, 32, within))

    PREPARE_INSIDE_ROWS = 16     # rows of a decode step up to which the attention kernel prepares q, k and v itself

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, x, residual, cache, then_norm=None):
        if cache is None:
            raise ValueError("attention needs a paged cache (its own, or the one it is told to read)")
        t, d, nq = rows_of(x), self.head_dim, self.num_heads
        nkv = 0 if self.kv_shared else self.num_kv_heads
        group = ctx.group(cache.group)
        qkv = ctx.scratch("attn_qkv", (t, (nq + 2 * nkv) * d), ctx.dtype)
        tables = self.position.tables(ctx)
        cos, sin = tables if tables is not None else (None, None)
        # 17..128 rows of a decode step: the q/k/v product and the preparation of its heads as two kernels, the
        # second adding up the sums of the product's K splits (no kernel of its own for that)
        together = (ctx.all_decode and self.b_qkv is None and ctx.dtype == torch.bfloat16 and t > self.PREPARE_INSIDE_ROWS
                    and ops.gemm_mid_qk_prep_takes(self.w_qkv.dtype, t, nq, nkv, d, self.w_qkv.shape[1], 0 if cos is None else cos.shape[1],
                                                   kernels_of(ctx)))
        begun = plain = None
        if together:
            begun = x if isinstance(x, ScaledRows) else None          # a norm that the product before began
            plain = begun.x if begun is not None else materialize(ctx, x)
            together = plain.dtype == torch.bfloat16 and plain.is_contiguous()
        if together:
            ops.gemm_mid_qk_prep(qkv, plain, self.w_qkv, None if begun is None else begun.sumsq, 0.0 if begun is None else begun.eps,
                                 nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin, cache.k_pages, cache.v_pages,
                                 group.slots, group.page_size, choice=kernels_of(ctx), workspace=workspace_of(ctx))
        else:
            linear(ctx, qkv, x if plain is None or begun is not None else plain, self.w_qkv, self.b_qkv)
        out = ctx.scratch("attn_out", (t, nq * d), ctx.dtype)
        kv_heads = cache.k_pages.shape[1]
        decode = ctx.all_decode and ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size)
        # a decode step's attention kernel normalises and rotates q and k and writes the new key and
        # value itself, when the rotation covers the whole head or there is none; beyond 16 rows a kernel
        # before it does that once a token (measured: 98 against 108 us for the attention kernel at 64 rows)
        whole_head = cos is None or cos.shape[1] * 2 == d
        prepare = queries_raw = None
        if together:
            pass
        elif decode and whole_head and ops.decode_prepare_supported(d, cos is not None) and t <= self.PREPARE_INSIDE_ROWS:
            prepare = ops.DecodePrepare(self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin, nkv)
        else:
            # a ragged step of heads of 128: the attention kernel normalises and rotates the q heads on their way into its
            # registers, so that only the k and v heads pass through a kernel before it (a third of the rows' bytes;
            # measured at 2,048 tokens, 32 q heads on 8: 19-22 -> 10.4 us for the kernel before attention, 66 -> 68 us
            # for attention itself)
            if (not decode and nkv > 0 and whole_head and ops.attention_prefill_prepares(d)
                    and ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size)):
                queries_raw = ops.DecodePrepare(self.q_norm, None, self.qk_norm_eps, cos, sin, 0)
            ops.qk_prep(qkv, nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin,
                        cache.k_pages, cache.v_pages, group.slots, group.page_size, skip_q=queries_raw is not None)
        if decode:
            longest, bound = ctx.max_k, ctx.max_k_bound
            if self.window is not None:
                longest, bound = min(longest, self.window + 32), min(bound, self.window + 64)
            splits = self._decode_splits(t * kv_heads, longest, bound, group.page_size)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.scratch("attn_part_o", (t, nq * splits * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t, nq * splits * 2), torch.float32)
            ops.attention_decode(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                                 nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, prepare,
                                 form=1)   # the next tile on its way while one is worked on, the first one before the query is prepared (measured: 0.6 % of a step)
        elif ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size):
            # sized by the step's coarse bound of the longest context, the same for every step of one shape
            longest = ctx.max_k_bound if self.window is None else min(ctx.max_k_bound, self.window + 64)
            singles = ctx.single_rows
            if singles:
                # the single tokens at the head of a mixed step (decoding requests beside a prompt portion) go to the
                # kernel of decode steps, which divides one token's keys between waves and workgroups; as rows of
                # the other kernel each would walk its whole context in one workgroup
                splits = self._decode_splits(singles * kv_heads, longest, ctx.max_k_bound, group.page_size)
                part_o = part_ml = None
                if splits > 1:
                    part_o = ctx.scratch("attn_single_part_o", (singles, nq * splits * d), torch.float32)
                    part_ml = ctx.scratch("attn_single_part_ml", (singles, nq * splits * 2), torch.float32)
                first = None
                if queries_raw is not None:      # the decode kernel prepares the q heads of its rows likewise
                    parted = None
                    if cos is not None:          # the tables' rows of the single tokens and of the rest, cut once a step
                        parted = ctx.memo.get(("rotation_rows", id(cos)))
                        if parted is None:
                            parted = ctx.memo[("rotation_rows", id(cos))] = (cos[:singles], sin[:singles], cos[singles:], sin[singles:])
                    first = ops.DecodePrepare(self.q_norm, self.k_norm, self.qk_norm_eps, None if parted is None else parted[0],
                                              None if parted is None else parted[1], 0)
                ops.attention_decode(out[:singles], qkv[:singles], cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot,
                                     ctx.positions, nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, first, form=1)
            rest = ctx.memo.get("rows_after_singles")
            if rest is None:
                rest = ctx.memo["rows_after_singles"] = (ctx.token_slot[singles:], ctx.positions[singles:])
            if queries_raw is not None and singles and cos is not None:
                queries_raw = ops.DecodePrepare(self.q_norm, None, self.qk_norm_eps, parted[2], parted[3], 0)
            splits = self._prefill_splits(ctx.num_qblocks * kv_heads, longest, (t - singles) * nq * d, nq // kv_heads, t - singles)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.scratch("attn_part_o", (t - singles, nq * splits * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t - singles, nq * splits * 2), torch.float32)
            ops.attention_prefill(out[singles:], qkv[singles:], cache.k_pages, cache.v_pages, group.block_table, rest[0], rest[1],
                                  ctx.qblock_token0, ctx.qblock_count, nq, self.scale, self.window or 0, ctx.max_qblock, ctx.max_k_bound,
                                  splits, part_o, part_ml, queries_raw)
        else:
            ops.attention(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                          nq, self.scale, self.window or 0)
        return linear(ctx, residual, out, self.w_o, accumulate=True, then_norm=then_norm)


register("mixer", "gqa_attention", GQAAttention)
