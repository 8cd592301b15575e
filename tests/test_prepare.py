"""The host routine that fills a step's metadata (csrc/prepare.hip) against the Python routine it replaces: random
steps of every kind (decode-only with and without padding, prepared ahead of later steps, prompt portions, mixed steps
with single tokens at the head or further back, places wanted twice, windowed groups whose early pages are gone) give
the same staging buffer word for word and the same numbers in the step's context.  No GPU needed: nothing is copied."""

import numpy as np
import pytest
import torch

from tests import toy_arch  # noqa: F401  (registers an architecture without attention, for a model that wants no query groups)
from tests.helpers import TINY_B


def make_runner(raw=TINY_B, page_size=16, requests=6, seq=512, step_tokens=300, window=None):
    import dataclasses

    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine.step import ModelRunner
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.parts import PartSpec

    spec = spec_for(config_from_dict(raw))
    if window is not None:          # a second cache group with a window: its early pages are given back
        block = spec.layers[0]
        windowed = PartSpec("prenorm", dict(block.params, mixer=PartSpec("gqa_attention", dict(block.params["mixer"].params, window=window))))
        spec = dataclasses.replace(spec, layers=(windowed,) + spec.layers[1:])
    model = DecoderModel(spec)
    cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=200, max_requests=requests, max_seq_len=seq, device="cpu",
                         allocate_storage=False)
    return ModelRunner(model, cache, max_step_tokens=step_tokens, dtype=torch.float32, device="cpu")


def both_ways(runner, entries, pad_to=0, ahead=0):
    from llm_runtime_study_amd.engine.step import StepContext

    results = []
    for native in (True, False):
        runner._off, runner._meta_size = runner._layout(max(sum(len(e.tokens) for e in entries), pad_to), max(len(entries), pad_to))
        runner._host_np[:] = -7                      # what a routine does not write stays recognisable
        ctx = StepContext(runner)
        (runner._prepare_native if native else runner._prepare_python)(ctx, entries, pad_to, ahead)
        used = {name: runner._host_view(name).copy() for name in runner._off}
        results.append((ctx, used))
    (a, words_a), (b, words_b) = results
    for name in ("T", "R", "num_logit_rows", "num_qblocks", "max_qblock", "max_q", "max_k", "single_rows", "host_q_lens", "host_slots", "host_positions"):
        assert getattr(a, name) == getattr(b, name), name
    written = {"token_ids": a.T, "positions": a.T, "token_request": a.T, "token_slot": a.T, "logit_rows": a.num_logit_rows,
               "cu_seqlens_q": a.R + 1, "seq_lens_k": a.R, "slot_ids": a.R, "qblock_token0": a.num_qblocks, "qblock_count": a.num_qblocks, "counts": 1}
    for name, values in words_a.items():
        count = written.get(name, a.T)               # the groups' slot arrays hold a value a token
        assert (values[:count] == words_b[name][:count]).all(), name
        assert (values[:count] != -7).all() or name in ("logit_rows",), name
    return a


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [None, 40])
def test_native_and_python_prepare_agree_on_random_steps(seed, window):
    from llm_runtime_study_amd.engine.step import StepEntry

    rng = np.random.default_rng(seed)
    runner = make_runner(window=window)
    cache = runner.cache
    vocab = TINY_B["vocab_size"]
    live = [cache.admit(i) for i in range(5)]
    for request in live:                             # contexts of very different lengths; some sit at a page's edge
        cache.extend(request, int(rng.choice([1, 15, 16, 17, 130, 257])))
        cache.trim(request)
    for turn in range(30):
        kind = turn % 5
        chosen = [live[i] for i in sorted(rng.choice(5, size=int(rng.integers(1, 6)), replace=False).tolist())]
        entries, before = [], [r.length for r in chosen]
        if kind in (0, 1):                           # decode-only, with or without padding, perhaps ahead of later steps
            ahead = int(rng.integers(0, 3)) if kind == 1 else 0
            for request in chosen:
                cache.extend(request, 1 + ahead)
                entries.append(StepEntry(request, [int(rng.integers(0, vocab))], [0] if rng.random() < 0.8 else []))
            pad = int(rng.choice([0, 8])) if kind == 0 else 8
            ctx = both_ways(runner, entries, pad_to=pad if pad >= len(entries) else 0, ahead=ahead)
            assert ctx.max_q == 1
        else:                                        # portions and mixed steps
            singles_first = kind == 2
            for place, request in enumerate(chosen):
                n = 1 if (singles_first and place < 2) or rng.random() < 0.25 else int(rng.integers(2, 50))
                cache.extend(request, n)
                want = sorted(rng.choice(n, size=int(rng.integers(0, min(n, 3) + 1)), replace=True).tolist())   # a place may come twice
                entries.append(StepEntry(request, rng.integers(0, vocab, n).tolist(), want))
            if all(len(e.tokens) == 1 for e in entries):
                cache.extend(chosen[-1], 5)
                entries[-1] = StepEntry(chosen[-1], rng.integers(0, vocab, 6).tolist(), [5])
            both_ways(runner, entries)
        for request, length in zip(chosen, before):  # some steps are taken back, the others stay
            if rng.random() < 0.3:
                cache.rollback(request, length)
            else:
                cache.trim(request)
            if request.length > 400:
                cache.rollback(request, 0) if window is None else None
        for i, request in enumerate(live):
            if request.length > 400:
                cache.release(request)
                live[i] = cache.admit(100 + turn * 10 + i)
                cache.extend(live[i], 3)
    cache.check_invariants()


def test_a_model_that_wants_no_query_groups_gets_none_from_either_routine():
    from llm_runtime_study_amd.engine.step import StepEntry

    runner = make_runner(raw=dict(toy_arch.TOY_MIX, pattern="mm"))
    cache = runner.cache
    a, b = cache.admit("a"), cache.admit("b")
    cache.extend(a, 1), cache.extend(b, 12)
    ctx = both_ways(runner, [StepEntry(a, [4], [0]), StepEntry(b, list(range(12)), [11, 3])])
    assert ctx.num_qblocks == 0 and ctx.max_qblock == 0 and ctx.single_rows == 0 and ctx.num_logit_rows == 3
