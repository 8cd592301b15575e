"""The step function's own promises: what it refuses, that a failing forward leaves no trace in the
caches (reference tests/test_cache.py:306-324, mini_llm/model/base.py:136-156,180-190), that decode
launches of several steps give the tokens of single steps also across a length class's edge, the
package's own many-rows product inside whole steps, and one layer at the benchmark's sizes against
the plain implementation directly."""

import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import TINY_B, TINY_C
from tests.plain import model as plain

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = tmp_path_factory.mktemp("step_b")
    write_model_dir(config_from_dict(TINY_B), seed=41, model_dir=folder, init="scaled")
    return folder


@pytest.fixture(scope="module")
def folder_heads_of_128(tmp_path_factory):
    """Heads of 128 dims, the size whose kernel for ragged steps prepares the queries itself; kv groups of three heads
    (a wave of the four has none), everything else small."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = tmp_path_factory.mktemp("step_heads_of_128")
    write_model_dir(config_from_dict(dict(TINY_C, head_dim=128, num_attention_heads=6, num_key_value_heads=2, vocab_size=290)),
                    seed=43, model_dir=folder, init="scaled")
    return folder


def make_runner(folder, dtype, *, pages=40, requests=4, seq=256, step_tokens=64, graph=False, page_size=16):
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner

    device = torch.device("cuda", 0)
    _, model = load_model(folder, dtype, device)
    cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=pages, max_requests=requests, max_seq_len=seq, dtype=dtype, device=device)
    return ModelRunner(model, cache, max_step_tokens=step_tokens, dtype=dtype, device=device, use_graph=graph)


def snapshot(cache, requests):
    """Everything a failed step must leave as it was."""
    return ([r.length for r in requests], [[list(t) for t in r.tables] for r in requests],
            [cache.used_pages(g) for g in range(len(cache.groups))], [cache.free_pages(g) for g in range(len(cache.groups))],
            [g.host_table.copy() for g in cache.groups], cache.active_requests)


def same(a, b):
    return a[:4] == b[:4] and all((x == y).all() for x, y in zip(a[4], b[4])) and a[5] == b[5]


class Failing(RuntimeError):
    pass


# ------------------------------------------------------------------ refusals
def test_every_refusal_of_the_step_function_leaves_the_cache_alone(folder_b):
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.errors import GenerationError

    runner = make_runner(folder_b, torch.float32, requests=2, step_tokens=12)
    cache = runner.cache
    a, b = cache.admit("a"), cache.admit("b")
    runner.step([StepEntry(a, [1, 2, 3], [])])
    outsider = make_runner(folder_b, torch.float32, requests=3).cache.admit("c")
    vocab = TINY_B["vocab_size"]
    cases = [
        ([], "at least one entry"),
        ([StepEntry(a, [1]), StepEntry(b, [2]), StepEntry(outsider, [3])], "3 requests but at most 2"),
        ([StepEntry(a, [1]), StepEntry(b, [])], "at least one token"),
        ([StepEntry(a, [1]), StepEntry(a, [2])], "only once"),
        ([StepEntry(a, [1, vocab])], rf"within vocabulary \[0, {vocab}\)"),
        ([StepEntry(a, [1, -1])], "within vocabulary"),
        ([StepEntry(a, [1, 2], [2])], "wanted place 2 is outside the entry's 2 tokens"),
        ([StepEntry(a, [1, 2], [-1])], "wanted place -1"),
        ([StepEntry(a, [1] * 7), StepEntry(b, [2] * 6)], "13 tokens but at most 12"),
    ]
    before = snapshot(cache, [a, b])
    for entries, message in cases:
        with pytest.raises(GenerationError, match=message):
            runner.step(entries)
        assert same(snapshot(cache, [a, b]), before)
    with pytest.raises(GenerationError, match="1..8 steps"):
        runner.decode_steps([StepEntry(a, [1])], 9)
    with pytest.raises(GenerationError, match="needs graphs"):
        runner.decode_steps([StepEntry(a, [1])], 2)       # this runner was built without graphs
    assert same(snapshot(cache, [a, b]), before)
    cache.check_invariants()
    # a cache that was given back is refused by the cache manager, and the other entry's growth is undone
    cache.release(b)
    from llm_runtime_study_amd.errors import KVCacheError
    with pytest.raises(KVCacheError, match="released"):
        runner.step([StepEntry(a, [4]), StepEntry(b, [5])])
    assert a.length == 3
    cache.check_invariants()


# ------------------------------------------------------- a forward that fails
@pytest.mark.parametrize("failure", [Failing, KeyboardInterrupt], ids=["error", "interrupt"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_failing_forward_leaves_no_trace_in_a_mixed_step(folder_b, dtype, failure):
    """Two running requests decode beside a new request's first portion; the second layer raises (an error, or
    an interrupt from the keyboard, which is no Exception).  Lengths, page lists, pool counts and host block
    tables are as before, the new request holds nothing, the recording of launches that was open is closed, and
    the same step run again (recorded anew) gives what a runner that never failed gives."""
    from llm_runtime_study_amd.engine.step import StepEntry

    rng = np.random.default_rng(3)
    prompts = [rng.integers(0, TINY_B["vocab_size"], n).tolist() for n in (31, 16, 20)]

    def drive(fail: bool):
        runner = make_runner(folder_b, dtype, pages=12)
        cache = runner.cache
        r0, r1 = cache.admit(0), cache.admit(1)
        runner.step([StepEntry(r0, prompts[0], []), StepEntry(r1, prompts[1], [])])     # r1 ends exactly at a page's edge
        r2 = cache.admit(2)
        entries = [StepEntry(r0, [7], [0]), StepEntry(r1, [9], [0]), StepEntry(r2, prompts[2], [19])]
        if fail:
            before = snapshot(cache, [r0, r1, r2])
            layer = runner.model.layers[1]
            original = layer.forward

            def broken(*args, **kwargs):
                raise failure("the second layer fails")

            layer.forward = broken
            with pytest.raises(failure):
                runner.step(entries)
            layer.forward = original
            recorded = runner.plan_recordings
            assert same(snapshot(cache, [r0, r1, r2]), before)
            assert r2.length == 0 and r2.tables == [[]] and cache.used_pages() == 3
            cache.check_invariants()
        first = runner.step(entries).clone()
        if fail:
            assert runner.use_plans and runner.plan_recordings == recorded + 1     # no recording was left open
        second = runner.step([StepEntry(r0, [1], [0]), StepEntry(r1, [2], [0]), StepEntry(r2, [3], [0])]).clone()
        cache.check_invariants()
        return first, second

    for got, want in zip(drive(True), drive(False)):
        assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_failing_launch_of_several_decode_steps_leaves_no_trace(folder_b, dtype):
    """decode_steps(4) takes the pages of all four positions before it runs; the third step's forward
    raises.  One request sits two tokens before a page's edge, so the launch had taken a page for it."""
    from llm_runtime_study_amd.engine.step import StepEntry

    rng = np.random.default_rng(4)
    prompts = [rng.integers(0, TINY_B["vocab_size"], n).tolist() for n in (30, 9, 17)]

    def drive(fail: bool):
        runner = make_runner(folder_b, dtype, pages=12, graph=True)
        cache = runner.cache
        with torch.cuda.stream(torch.cuda.Stream(runner.device)):
            requests = [cache.admit(i) for i in range(3)]
            runner.step([StepEntry(r, p, []) for r, p in zip(requests, prompts)])
            entries = [StepEntry(r, [5 + i], [0]) for i, r in enumerate(requests)]
            assert runner.can_decode_steps(entries)
            if fail:
                before = snapshot(cache, requests)
                original, calls = runner.model.forward_hidden, []

                def broken(ctx):
                    calls.append(1)
                    if len(calls) == 3:
                        raise Failing("the third step fails")
                    return original(ctx)

                runner.model.forward_hidden = broken
                with pytest.raises(Failing):
                    runner.decode_steps(entries, 4)
                runner.model.forward_hidden = original
                assert len(calls) == 3 and same(snapshot(cache, requests), before)
                assert [r.length for r in requests] == [30, 9, 17] and cache.used_pages() == 2 + 1 + 2
                cache.check_invariants()
            chosen = runner.decode_steps(entries, 4)
            assert [r.length for r in requests] == [34, 13, 21]
            after = runner.step([StepEntry(r, [row], [0]) for r, row in zip(requests, chosen[-1])]).clone()
            torch.cuda.synchronize()          # the comparison below runs on another stream
            runner.drop_graphs()
        cache.check_invariants()
        return chosen, after

    (chosen, after), (chosen_ok, after_ok) = drive(True), drive(False)
    assert chosen == chosen_ok and torch.equal(after, after_ok)


# ------------------------------------------- launches that cross a class's edge
@pytest.mark.parametrize("dtype", DTYPES)
def test_tokens_do_not_depend_on_steps_per_launch_across_a_length_class_edge(tmp_path, dtype):
    """From a context of 254 tokens on, eight tokens in launches of 4, of 3 and one by one: the contexts
    cross 256, where decode attention begins to divide the keys.  Same tokens, same logits afterwards,
    same keys and values in the pages."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.weights import write_model_dir

    folder = tmp_path / "c"
    write_model_dir(config_from_dict(TINY_C), seed=42, model_dir=folder, init="scaled")
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, TINY_C["vocab_size"], n).tolist() for n in (253, 120)]
    outcomes = []
    for per_launch in (4, 3, 1):
        runner = make_runner(folder, dtype, pages=40, seq=320, step_tokens=512, graph=True)
        cache = runner.cache
        with torch.cuda.stream(torch.cuda.Stream(runner.device)):
            requests = [cache.admit(i) for i in range(2)]
            runner.step([StepEntry(r, p, []) for r, p in zip(requests, prompts)])
            tokens, last = [], [11, 12]
            while len(tokens) < 8:
                n = min(per_launch, 8 - len(tokens))
                chosen = runner.decode_steps([StepEntry(r, [t], [0]) for r, t in zip(requests, last)], n)
                tokens += chosen
                last = chosen[-1]
            final = runner.step([StepEntry(r, [t], [0]) for r, t in zip(requests, last)]).clone()
            torch.cuda.synchronize()
            layer = cache.layer_caches[1]
            pages = [p for r in requests for p in r.tables[0]]
            outcomes.append((tokens, final, layer.k_pages[pages].clone(), layer.v_pages[pages].clone(), pages))
            assert requests[0].length == 253 + 9 and runner.graph_replays + runner.graph_captures >= 8 // per_launch
            runner.drop_graphs()
    for tokens, final, keys, values, pages in outcomes[1:]:
        assert tokens == outcomes[0][0] and pages == outcomes[0][4]
        assert torch.equal(final, outcomes[0][1]) and torch.equal(keys, outcomes[0][2]) and torch.equal(values, outcomes[0][3])


# ---------------------------------------- the package's own many-rows product
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_through_the_own_many_rows_product(folder_b, dtype, tmp_path):
    """Replay with `library_gemm=False`: a 300-token prompt whole (more rows than the kernels for few
    rows take) and the same prompt in two portions, against the plain implementation."""
    from llm_runtime_study_amd.engine import trace

    cfg, weights = plain.load_model_dir(folder_b, torch.float64)
    rng = np.random.default_rng(8)
    requests = {"long": rng.integers(0, cfg["vocab_size"], 300).tolist(), "mid": rng.integers(0, cfg["vocab_size"], 150).tolist()}
    want = {key: plain.qwen3_forward(weights, cfg, ids) for key, ids in requests.items()}
    steps = traces.whole(requests)
    ids = requests["long"]
    steps += [{"step": len(steps), "entries": [{"id": "again", "tokens": ids[:170], "want": [0, 169]}], "end": []},
              {"step": len(steps) + 1, "entries": [{"id": "again", "tokens": ids[170:], "want": list(range(130))}], "end": ["again"]}]
    want["again"] = want["long"]
    runner = trace.make_runner(folder_b, dtype, 320, library_gemm=False)
    assert runner.library_gemm is False
    out = tmp_path / "logits"
    trace.replay(runner, traces.strip(steps).splitlines(), out, echo=lambda _: None)
    got = traces.collect(steps, out, cfg["vocab_size"])
    checked = 0
    for key, rows in got.items():
        for position, row in rows.items():
            ref = want[key][position]
            if dtype == "float32":
                torch.testing.assert_close(row.double(), ref, rtol=1e-4, atol=1e-4, msg=lambda m: f"{key}@{position}: {m}")
            else:
                err = (row.double() - ref).norm() / ref.norm()
                assert err < 3e-2, f"{key}@{position}: relative error {err:.3g}"
            checked += 1
    assert checked == 300 + 150 + 2 + 130


@pytest.mark.parametrize("model", ["b", "heads_of_128"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_single_tokens_at_the_head_of_a_mixed_step_and_elsewhere_in_it(folder_b, folder_heads_of_128, model, dtype, tmp_path):
    """Decoding requests beside a prompt portion: the single tokens that a step begins with go to the
    attention kernel of decode steps, single tokens further back stay rows of the other kernel, and one
    token that is a whole portion (a request's first) is a single token like any other.  Every asked row
    against the plain implementation.  (With heads of 128 dims both kernels take the raw q heads of the
    q/k/v product in bfloat16 and prepare them themselves.)"""
    from llm_runtime_study_amd.engine import trace

    folder_b = folder_b if model == "b" else folder_heads_of_128
    cfg, weights = plain.load_model_dir(folder_b, torch.float64)
    rng = np.random.default_rng(21)
    requests = {key: rng.integers(0, cfg["vocab_size"], n).tolist() for key, n in (("a", 45), ("b", 30), ("c", 64), ("d", 3))}
    want = {key: plain.qwen3_forward(weights, cfg, ids) for key, ids in requests.items()}
    a, b, c, d = (requests[key] for key in "abcd")

    def entry(key, tokens, first):
        return {"id": key, "tokens": tokens, "want": list(range(len(tokens)))}, [(key, first + i) for i in range(len(tokens))]

    plan = [
        [entry("a", a[:40], 0), entry("b", b[:25], 0)],
        [entry("a", a[40:41], 40), entry("b", b[25:26], 25), entry("c", c[:50], 0), entry("d", d[:1], 0)],      # two at the head, one at the end
        [entry("d", d[1:2], 1), entry("c", c[50:60], 50), entry("a", a[41:42], 41), entry("b", b[26:28], 26)],   # the head is a request's second token
        [entry("b", b[28:29], 28), entry("a", a[42:43], 42), entry("d", d[2:3], 2), entry("c", c[60:64], 60)],   # three single tokens, then a portion
    ]
    steps = [{"step": i, "entries": [e for e, _ in row], "end": []} for i, row in enumerate(plan)]
    runner = trace.make_runner(folder_b, dtype, 256)
    out = tmp_path / "logits"
    trace.replay(runner, traces.strip(steps).splitlines(), out, echo=lambda _: None)
    checked = 0
    for i, row in enumerate(plan):
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"]).copy())
        places = [place for _, where in row for place in where]
        assert got.shape[0] == len(places)
        for logits, (key, position) in zip(got, places):
            ref = want[key][position]
            if dtype == "float32":
                torch.testing.assert_close(logits.double(), ref, rtol=1e-4, atol=1e-4, msg=lambda m: f"step {i} {key}@{position}: {m}")
            else:
                err = (logits.double() - ref).norm() / ref.norm()
                assert err < 3e-2, f"step {i} {key}@{position}: relative error {err:.3g}"
            checked += 1
    assert checked == 65 + 53 + 14 + 7


# ------------------------------- one layer at the benchmark's sizes, against plain
@pytest.mark.parametrize("sizes", ["8b", "14b", "32b"])
def test_one_layer_at_the_benchmark_sizes_against_the_plain_implementation(sizes):
    """Hidden 4096, 32 query and 8 kv heads of 128 dims, feed-forward 12288, vocabulary 151936, float32,
    100 tokens in portions of 60, 39 and 1: the engine against the plain implementation itself, not against
    another precision of the engine.  The plain side computes the logits of three slices of the vocabulary
    (its first, a middle and its last rows) to keep the float64 work small.  Likewise at the layer sizes of the
    two larger models of the family (hidden 5120 with kv groups of five and of eight query heads), on which the
    comparison of the bfloat16 path with the float32 path at those sizes stands."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.weights import random_init
    from tests.test_shape_gpu import LARGER, SHAPE

    raw = dict(SHAPE, num_hidden_layers=1, **LARGER[sizes])
    cfg = config_from_dict(raw)
    device = torch.device("cuda", 0)
    model = DecoderModel(spec_for(cfg))
    weights = random_init.device_weights(model, 3, torch.bfloat16, device, "scaled")
    model.bind(weights, torch.float32)
    cache = CacheManager(model.cache_needs(), page_size=16, num_pages=8, max_requests=1, max_seq_len=128, dtype=torch.float32, device=device)
    runner = ModelRunner(model, cache, max_step_tokens=128, dtype=torch.float32, device=device)
    rng = np.random.default_rng(9)
    ids = rng.integers(0, cfg.vocab_size, 100).tolist()
    request = cache.admit("r")
    rows = []
    for portion in (ids[:60], ids[60:99], ids[99:]):
        rows.append(runner.step([StepEntry(request, portion, list(range(len(portion))))]).cpu())
    got = torch.cat(rows)
    # the plain side: only the embedding rows and head rows it needs, in float64
    vocab = cfg.vocab_size
    columns = torch.cat([torch.arange(0, 700), torch.arange(70000, 70700), torch.arange(vocab - 700, vocab)])
    used = sorted(set(ids))
    small = {name: t.cpu().double() for name, t in weights.items() if name not in ("model.embed_tokens.weight", "lm_head.weight")}
    small["model.embed_tokens.weight"] = weights["model.embed_tokens.weight"][torch.tensor(used, device=device)].cpu().double()
    small["lm_head.weight"] = weights["lm_head.weight"][columns.to(device)].cpu().double()
    want = plain.qwen3_forward(small, raw, [used.index(t) for t in ids])
    torch.testing.assert_close(got[:, columns].double(), want, rtol=1e-4, atol=1e-4)
    assert want.abs().max() > 1.0


@pytest.mark.parametrize("sizes,batch", [("14b", 40), ("32b", 64), ("8b", 33)])
def test_decode_steps_of_17_to_64_rows_at_the_benchmark_sizes_against_the_plain_implementation(sizes, batch):
    """One layer at the sizes of the family's larger models in bfloat16, decode steps of 33..64 requests: the products
    of 17..64 rows as the runner chooses them there (weight rows dealt evenly over the compute units with an extra
    tile for some workgroups, K divided for the narrow matrices, the norms taken apart around them) and decode
    attention over caches of different lengths, against the plain implementation on three slices of the vocabulary."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.weights import random_init
    from tests.test_shape_gpu import LARGER, SHAPE

    raw = dict(SHAPE, num_hidden_layers=1, **LARGER[sizes])
    cfg = config_from_dict(raw)
    device = torch.device("cuda", 0)
    model = DecoderModel(spec_for(cfg))
    weights = random_init.device_weights(model, 4, torch.bfloat16, device, "scaled")
    model.bind(weights, torch.bfloat16)
    cache = CacheManager(model.cache_needs(), page_size=16, num_pages=2 * batch, max_requests=batch, max_seq_len=32, dtype=torch.bfloat16, device=device)
    runner = ModelRunner(model, cache, max_step_tokens=1024, dtype=torch.bfloat16, device=device)
    rng = np.random.default_rng(11)
    prompts = [rng.integers(0, cfg.vocab_size, int(rng.integers(2, 13))).tolist() for _ in range(batch)]
    decoded = [rng.integers(0, cfg.vocab_size, 3).tolist() for _ in range(batch)]
    requests = [cache.admit(i) for i in range(batch)]
    runner.step([StepEntry(r, p, []) for r, p in zip(requests, prompts)])
    got = [runner.step([StepEntry(r, [d[i]], [0]) for r, d in zip(requests, decoded)]).cpu() for i in range(3)]   # [3][batch, vocab]
    vocab = cfg.vocab_size
    columns = torch.cat([torch.arange(0, 500), torch.arange(70000, 70500), torch.arange(vocab - 500, vocab)])
    used = sorted({t for seq in prompts + decoded for t in seq})
    small = {name: t.cpu().double() for name, t in weights.items() if name not in ("model.embed_tokens.weight", "lm_head.weight")}
    small["model.embed_tokens.weight"] = weights["model.embed_tokens.weight"][torch.tensor(used, device=device)].cpu().double()
    small["lm_head.weight"] = weights["lm_head.weight"][columns.to(device)].cpu().double()
    worst = 0.0
    for index, (prompt, more) in enumerate(zip(prompts, decoded)):
        want = plain.qwen3_forward(small, raw, [used.index(t) for t in prompt + more])
        for i in range(3):
            ref, mine = want[len(prompt) + i], got[i][index, columns].double()
            err = float((mine - ref).norm() / ref.norm())
            worst = max(worst, err)
            assert err < 3e-2, f"request {index}, decode step {i}: relative error {err:.3g}"
    assert worst > 0


# ------------------------------------------- launches that follow each other
@pytest.mark.parametrize("sampled", [False, True], ids=["greedy", "drawn"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_launches_that_follow_each_other_give_the_tokens_of_single_steps(tmp_path, dtype, sampled):
    """Launches of decode steps queued one behind the other, each begun before the one before is read (the device
    feeds itself, the host sends only new pages' table entries), against decode_steps() one launch at a time: the
    same tokens, across page edges and the edge of a length class (one request grows past 256 tokens), greedy and
    with seeded draws; the caches end as long, and a step after the chain sees what it left."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.sampling import SamplingConfig, SamplingRow
    from llm_runtime_study_amd.weights import write_model_dir

    folder = tmp_path / "model"
    write_model_dir(config_from_dict(TINY_C), seed=47, model_dir=folder, init="scaled")
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, TINY_C["vocab_size"], n).tolist() for n in (242, 30, 9)]
    configs = [SamplingConfig(temperature=0.9, top_k=40, seed=5), SamplingConfig(), SamplingConfig(temperature=0.7, top_p=0.8, seed=6)]

    def rows(produced):
        return [SamplingRow(c, c.seed or 0, produced) for c in configs] if sampled else None

    def drive(chained: bool):
        runner = make_runner(folder, dtype, pages=40, requests=3, seq=320, step_tokens=320, graph=True)
        cache = runner.cache
        with torch.cuda.stream(torch.cuda.Stream(runner.device)):
            requests = [cache.admit(i) for i in range(3)]
            first = runner.step([StepEntry(r, p, [len(p) - 1]) for r, p in zip(requests, prompts)]).argmax(-1).tolist()
            entries = [StepEntry(r, [t], [0]) for r, t in zip(requests, first)]
            tokens = []
            if chained:
                launches = [runner.decode_launch_begin(entries, 4, rows(0))]
                for _ in range(6):
                    launches.append(runner.decode_launch_begin(entries, 4, rows(0), after=launches[-1]))
                    tokens += runner.decode_launch_end(launches[-2])
                tokens += runner.decode_launch_end(launches[-1])
                assert all(launch.ended for launch in launches) and sum(launch.steps for launch in launches) == len(tokens)
                assert any(launch.steps < 4 for launch in launches)          # one ended at the edge of the length class
            else:
                while len(tokens) < 22:
                    latest = [StepEntry(r, [t], [0]) for r, t in zip(requests, tokens[-1])] if tokens else entries
                    tokens += runner.decode_steps(latest, min(4, 22 - len(tokens)), rows(len(tokens)))
            lengths = [r.length - len(tokens) for r in requests]          # every cache grew by what was decoded
            after = runner.step([StepEntry(r, [t], [0]) for r, t in zip(requests, tokens[-1])]).argmax(-1).tolist()
            tokens = tokens[:22]
            torch.cuda.synchronize()
            assert cache.tables_match_device()
            runner.drop_graphs()
        cache.check_invariants()
        return tokens, lengths, after

    chained, chained_lengths, after_chain = drive(True)
    single, single_lengths, _ = drive(False)
    assert chained == single and len(chained) == 22
    assert chained_lengths == single_lengths == [len(p) for p in prompts]
    assert all(0 <= t < TINY_C["vocab_size"] for t in after_chain)            # a step after the chain runs on what it left
    if sampled:
        assert len({tuple(row) for row in chained}) > 5                      # draws, not a fixed point


def test_a_launch_follows_only_the_launch_begun_last(folder_b):
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.errors import GenerationError

    runner = make_runner(folder_b, torch.float32, pages=12, graph=True)
    cache = runner.cache
    with torch.cuda.stream(torch.cuda.Stream(runner.device)):
        a, b = cache.admit("a"), cache.admit("b")
        runner.step([StepEntry(a, [3, 4, 5], []), StepEntry(b, [6], [])])
        entries = [StepEntry(a, [7], [0]), StepEntry(b, [8], [0])]
        first = runner.decode_launch_begin(entries, 2)
        with pytest.raises(GenerationError, match="same requests in the same order"):
            runner.decode_launch_begin(entries[::-1], 2, after=first)
        assert [a.length, b.length] == [5, 3]                                # the refused launch took nothing
        second = runner.decode_launch_begin(entries, 2, after=first)
        tokens = runner.decode_launch_end(first) + runner.decode_launch_end(second)
        assert len(tokens) == 4 and [a.length, b.length] == [7, 5]
        runner.step([StepEntry(a, [tokens[-1][0]], [0])])                     # another step: the device's metadata is its own now
        with pytest.raises(GenerationError, match="begun last"):
            runner.decode_launch_begin(entries, 2, after=second)
        with pytest.raises(GenerationError, match="ended before"):
            runner.decode_launch_end(second)
        torch.cuda.synchronize()
        runner.drop_graphs()
    cache.check_invariants()


# ------------------------------------------------ block tables that stay on the device
@pytest.mark.parametrize("dtype", DTYPES)
def test_block_tables_on_the_device_follow_the_hosts(folder_b, dtype):
    """The device keeps the block tables; a step sends only the entries that changed since the last one.  Through
    prompts, decoding, a rollback, a release and a new request in the freed slot the device's tables equal the
    host's after every step, also when a step has more changes than its metadata has room for (then the whole
    tables are sent), and the logits equal those of a runner that never ran short of room."""
    from llm_runtime_study_amd.engine.step import StepEntry

    rng = np.random.default_rng(23)
    vocab = TINY_B["vocab_size"]
    tokens = {key: rng.integers(0, vocab, n).tolist() for key, n in (("a", 150), ("b", 40), ("c", 90))}
    outs = []
    for room in (2048, 3):
        runner = make_runner(folder_b, dtype, pages=48, requests=2, seq=256, step_tokens=160, page_size=8)
        runner.TABLE_PATCHES = room
        cache = runner.cache
        rows = []
        a, b = cache.admit("a"), cache.admit("b")
        rows.append(runner.step([StepEntry(a, tokens["a"][:100], [99]), StepEntry(b, tokens["b"][:33], [32])]).clone())
        assert cache.tables_match_device()
        for i in range(7):                         # b crosses a page's edge while decoding
            rows.append(runner.step([StepEntry(a, [tokens["a"][100 + i]], [0]), StepEntry(b, [tokens["b"][33 + i]], [0])]).clone())
            assert cache.tables_match_device()
        cache.extend(a, 20)                        # pages taken and given back without a step between
        cache.rollback(a, 107)
        cache.release(b)
        c = cache.admit("c")                       # b's slot and, lowest ids first, b's pages
        assert c.slot == b.slot
        rows.append(runner.step([StepEntry(a, tokens["a"][107:150], [42]), StepEntry(c, tokens["c"], [89])]).clone())
        assert cache.tables_match_device() and not cache._dirty
        cache.check_invariants()
        outs.append(torch.cat(rows))
    assert torch.equal(outs[0], outs[1])
    cfg, weights = plain.load_model_dir(folder_b, torch.float64)
    want_a, want_c = plain.qwen3_forward(weights, cfg, tokens["a"]), plain.qwen3_forward(weights, cfg, tokens["c"])
    for got, want in ((outs[0][0], want_a[99]), (outs[0][-2], want_a[149]), (outs[0][-1], want_c[89])):
        err = (got.double().cpu() - want).norm() / want.norm()
        assert err < (1e-5 if dtype == torch.float32 else 3e-2)


# ---------------------------------------------------------------- launch plans
@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_made_again_from_a_recorded_plan_equal_steps_through_the_parts(folder_b, dtype):
    """Two runners over the same weights, one recording launch plans, one not, through the same steps: prompt
    portions, mixed steps and eager decode steps whose shapes come back with other tokens, other pages and
    other (longer) contexts.  Every logits row and the pages are bit for bit the same; the second time a
    shape comes, it is served from the plan; a shape whose longest context has left its 256-token class is
    recorded anew."""
    from llm_runtime_study_amd.engine.step import StepEntry

    rng = np.random.default_rng(11)
    vocab = TINY_B["vocab_size"]
    runners = [make_runner(folder_b, dtype, pages=80, requests=4, seq=400, step_tokens=96) for _ in range(2)]
    runners[1].use_plans = False
    assert runners[0].use_plans
    caches = [[r.cache.admit(i) for i in range(4)] for r in runners]

    def both(plan):
        """plan: list of (request, tokens, want); runs it on both runners and compares."""
        outs = []
        for runner, mine in zip(runners, caches):
            outs.append(runner.step([StepEntry(mine[i], tokens, want) for i, tokens, want in plan]))
        if outs[0] is None:
            assert outs[1] is None
        else:
            assert torch.equal(outs[0], outs[1])

    def portion(n):
        return rng.integers(0, vocab, n).tolist()

    # rounds one and two: every shape is new; a step during which a scratch buffer was made or grown is not kept
    # (addresses written down before the buffer moved are stale), so a shape may be recorded twice
    for first, second, third in ((0, 1, 2), (3, 2, 1)):
        both([(first, portion(40), [39]), (second, portion(33), [0, 32])])
        both([(first, portion(1), [0]), (second, portion(1), [0]), (third, portion(20), [19])])
        both([(0, portion(1), [0]), (1, portion(1), [0]), (2, portion(1), [0])])
    recorded, replayed = runners[0].plan_recordings, runners[0].plan_replays
    assert recorded == 3 and 1 <= replayed <= 3 and len(runners[0]._plans) == 3      # a recording that was not kept counts as neither
    # round three: the same shapes with other tokens, requests in other places and longer contexts (still below 256)
    both([(2, portion(40), [39]), (3, portion(33), [0, 32])])
    both([(2, portion(1), [0]), (3, portion(1), [0]), (0, portion(20), [19])])
    for _ in range(5):
        both([(0, portion(1), [0]), (1, portion(1), [0]), (2, portion(1), [0])])
    assert runners[0].plan_recordings == recorded and runners[0].plan_replays == replayed + 7
    # request 1 grows past 256 tokens: the same three-token decode shape, another class of context, a new plan
    both([(1, portion(96), [])])
    both([(1, portion(96), [95])])
    both([(1, portion(30), [])])
    assert caches[0][1].length > 256
    before = runners[0].plan_recordings
    both([(0, portion(1), [0]), (1, portion(1), [0]), (2, portion(1), [0])])
    both([(0, portion(1), [0]), (1, portion(1), [0]), (2, portion(1), [0])])
    assert runners[0].plan_recordings == before + 1
    torch.cuda.synchronize()
    for a, b in zip(runners[0].cache.layer_caches, runners[1].cache.layer_caches):
        assert torch.equal(a.k_pages, b.k_pages) and torch.equal(a.v_pages, b.v_pages)
    # a model with a part that is not known to be safe to record runs through its parts every time
    runners[0].cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_graph_of_a_plan_equals_the_parts_and_the_plain_implementation(folder_b, dtype):
    """The path steady serving runs on: a step shape that keeps coming back on a stream of its own is recorded,
    replayed from the plan and then launched as the graph of that plan.  One mixed shape (two requests bringing a
    single token, a third a portion of 20) comes eleven times, with other tokens, requests changing roles, contexts
    growing, and pages that a finished request gave back and a new one took.  Every logits row equals, bit for bit,
    that of a runner without plans through the same steps, and agrees with the plain implementation of the whole
    sequences."""
    from llm_runtime_study_amd.engine.step import StepEntry

    cfg, weights = plain.load_model_dir(folder_b, torch.float64)
    rng = np.random.default_rng(17)
    vocab = TINY_B["vocab_size"]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        runners = [make_runner(folder_b, dtype, pages=40, requests=3, seq=256, step_tokens=32) for _ in range(2)]
        runners[1].use_plans = False
        assert runners[0].use_plans
        caches = [[r.cache.admit(i) for i in range(3)] for r in runners]
        history = {0: [], 1: [], 2: []}            # request -> its tokens so far
        names = [0, 1, 2]                          # which request sits in each of the three places
        finished, got = {}, {}
        rounds = runners[0].PLAN_GRAPH_AFTER + 8
        for turn in range(rounds):
            if turn == 6:
                # the request in place 0 ends; a new one takes its slot and, lowest ids first, other pages than it had
                finished[names[0]] = history.pop(names[0])
                for runner, mine in zip(runners, caches):
                    runner.cache.release(mine[0])
                    mine[0] = runner.cache.admit(3)
                names[0], history[3] = 3, []
            singles, portion = [(turn + 0) % 3, (turn + 1) % 3], (turn + 2) % 3
            plan = [(place, rng.integers(0, vocab, 1).tolist(), [0]) for place in singles]
            plan.append((portion, rng.integers(0, vocab, 20).tolist(), [3, 19]))
            outs = []
            for runner, mine in zip(runners, caches):
                outs.append(runner.step([StepEntry(mine[place], tokens, want) for place, tokens, want in plan]).clone())
            assert torch.equal(outs[0], outs[1]), f"turn {turn}"
            row = 0
            for place, tokens, want in plan:
                at = len(history[names[place]])
                for w in want:
                    got[(names[place], at + w)] = outs[0][row].cpu()
                    row += 1
                history[names[place]] += tokens
        side.synchronize()
        known = [k for k in runners[0]._plans.values() if k.graph is not None]
        assert len(known) == 1 and runners[0].plan_recordings <= 3
        assert runners[0].plan_graph_replays >= rounds - 3 - runners[0].PLAN_GRAPH_AFTER
        assert runners[1].plan_replays == 0
        for a, b in zip(runners[0].cache.layer_caches, runners[1].cache.layer_caches):
            assert torch.equal(a.k_pages, b.k_pages) and torch.equal(a.v_pages, b.v_pages)
    finished.update(history)
    want = {name: plain.qwen3_forward(weights, cfg, ids) for name, ids in finished.items()}
    assert len(got) == rounds * 4
    for (name, position), row in got.items():
        ref = want[name][position]
        if dtype == torch.float32:
            torch.testing.assert_close(row.double(), ref, rtol=1e-4, atol=1e-4, msg=lambda m: f"request {name} position {position}: {m}")
        else:
            err = (row.double() - ref).norm() / ref.norm()
            assert err < 3e-2, f"request {name} position {position}: relative error {err:.3g}"
            assert int(row.argmax()) == int(ref.argmax()) or ref.topk(2).values.diff().abs() < 0.25


def test_a_model_with_parts_of_unknown_habits_is_never_recorded():
    from tests.test_parts_gpu import RunningMeanMixer, build_runner, toy_state_model

    spec, weights, _, _ = toy_state_model("toy_running_mean", RunningMeanMixer)
    runner = build_runner(spec, weights, torch.float32)
    assert not runner.use_plans
