"""The engine as a user meets it: greedy generation through the entry point, long decoding,
the first tokens of a sequence, graph replay against eager steps, seeded sampling, a pool so
small that requests wait, and the command line."""

import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import TINY_A, TINY_B, TINY_C
from tests.plain import model as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    out = {}
    for name, raw, seed in (("a", TINY_A, 31), ("b", TINY_B, 32), ("c", TINY_C, 33)):
        folder = tmp_path_factory.mktemp(f"engine_{name}")
        write_model_dir(config_from_dict(raw), seed=seed, model_dir=folder, init="scaled")
        cfg, weights = plain.load_model_dir(folder, torch.float64)
        out[name] = (folder, cfg, weights)
    return out


def plain_greedy(cfg, weights, prompt, new_tokens, stop=()):
    ids = list(prompt)
    for _ in range(new_tokens):
        ids.append(int(plain.qwen3_forward(weights, cfg, ids)[-1].argmax()))
        if ids[-1] in stop:
            break
    return ids[len(prompt):]


@pytest.mark.parametrize("name", ["a", "b", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    from llm_runtime_study_amd import Engine, SamplingConfig

    folder, cfg, weights = folders[name]
    rng = np.random.default_rng(4)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (5, 11, 17, 1, 40)]
    eos = cfg["eos_token_id"] if isinstance(cfg["eos_token_id"], list) else [cfg["eos_token_id"]]
    expected = [plain_greedy(cfg, weights, p, 8, eos) for p in prompts]
    engine = Engine.from_model_dir(folder, dtype=dtype, max_seq_len=96, max_batch_size=3, max_num_batched_tokens=16)
    events = list(engine.generate(prompts, max_new_tokens=8, sampling=SamplingConfig()))
    got = [[e.token_id for i, e in events if i == r] for r in range(len(prompts))]
    if dtype == "float32":
        assert got == expected
    else:
        same = sum(a == b for g, e in zip(got, expected) for a, b in zip(g, e))
        assert same >= 0.85 * sum(len(e) for e in expected)
    firsts = [e for _, e in events if e.prompt_token_count is not None]
    assert sorted(e.prompt_token_count for e in firsts) == sorted(len(p) for p in prompts)
    for r in range(len(prompts)):
        last = [e for i, e in events if i == r][-1]
        assert last.finish_reason == ("eos" if last.token_id in eos else "max_new_tokens")
    assert all(e.model_seconds is not None and e.model_seconds > 0 for _, e in events)
    manager = engine.cache_manager
    manager.check_invariants()
    assert manager.active_requests == 0 and manager.used_pages() == 0
    assert engine.last_cache_capacity == len(prompts[-1]) + 8 and engine.last_cache_num_bytes > 0


@pytest.mark.parametrize("name", ["b", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_token_by_token(folders, name, dtype, tmp_path):
    """8 prompt tokens, then 400 tokens one by one: every logits row against the plain model."""
    from llm_runtime_study_amd.engine import trace

    folder, cfg, weights = folders[name]
    ids = np.random.default_rng(6).integers(0, cfg["vocab_size"], 408).tolist()
    want = plain.qwen3_forward(weights, cfg, ids)
    steps = traces.prefill_then_decode({"r": ids}, tail=400)
    runner = trace.make_runner(folder, dtype, 448)
    trace.replay(runner, traces.strip(steps).splitlines(), tmp_path, echo=lambda _: None)
    got = traces.collect(steps, tmp_path, cfg["vocab_size"])["r"]
    assert len(got) == 408
    for position, row in got.items():
        if dtype == "float32":
            torch.testing.assert_close(row.double(), want[position], rtol=1e-4, atol=1e-4, msg=lambda m: f"position {position}: {m}")
        else:
            err = (row.double() - want[position]).norm() / want[position].norm()
            assert err < 3e-2, f"position {position}: relative error {err:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence_one_by_one(folders, dtype, tmp_path):
    from llm_runtime_study_amd.engine import trace

    folder, cfg, weights = folders["a"]
    ids = [9, 200, 3, 77, 150, 4]
    want = plain.qwen3_forward(weights, cfg, ids)
    steps = [{"step": i, "entries": [{"id": "r", "tokens": [t], "want": [0]}], "end": ["r"] if i == 5 else []} for i, t in enumerate(ids)]
    runner = trace.make_runner(folder, dtype, 64)
    trace.replay(runner, traces.strip(steps).splitlines(), tmp_path, echo=lambda _: None)
    got = traces.collect(steps, tmp_path, cfg["vocab_size"])["r"]
    for position in range(6):
        err = (got[position].double() - want[position]).norm() / want[position].norm()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"position {position}: {err:.3g}"


@pytest.mark.parametrize("lengths", [(3, 30, 17, 45, 9), (3, 250, 17, 500, 9)], ids=["short", "crossing-split-classes"])
@pytest.mark.parametrize("name", ["b", "c"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graph_replay_equals_eager_steps(folders, name, dtype, lengths):
    """Decode steps through captured graphs, with eager prefill work and synchronisations between the
    replays; every replay's logits must equal those of the same step run eagerly. The longer prompts
    grow past 256 and 512 tokens while decoding, where decode attention starts to divide the keys
    among more workgroups and a graph captured for the shorter context must not be replayed."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry

    folder, cfg, _ = folders[name]
    device = torch.device("cuda", 0)
    _, model = load_model(folder, dtype, device)
    rng = np.random.default_rng(8)

    def make(use_graph):
        cache = CacheManager(model.cache_needs(), page_size=16, num_pages=40 + sum(lengths) // 16, max_requests=8, max_seq_len=1024,
                             dtype=dtype, device=device)
        return ModelRunner(model, cache, max_step_tokens=512, dtype=dtype, device=device, use_graph=use_graph)

    eager, graphed = make(False), make(True)
    assert graphed.use_graph
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in lengths]
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        live = {}
        for step in range(24):
            if step in (0, 1, 5, 9, 13):       # a new request joins: an eager prefill step between replays
                index = len(live)
                caches = (eager.cache.admit(index), graphed.cache.admit(index))
                a = eager.step([StepEntry(caches[0], prompts[index], [len(prompts[index]) - 1])]).clone()
                b = graphed.step([StepEntry(caches[1], prompts[index], [len(prompts[index]) - 1])]).clone()
                assert torch.equal(a, b)
                live[index] = (caches, int(a[0].argmax()))
            if step == 17:                      # a request leaves: the batch shrinks to another bucket
                caches, _ = live.pop(1)
                eager.cache.release(caches[0])
                graphed.cache.release(caches[1])
            order = sorted(live)
            a = eager.step([StepEntry(live[i][0][0], [live[i][1]], [0]) for i in order]).clone()
            b = graphed.step([StepEntry(live[i][0][1], [live[i][1]], [0]) for i in order]).clone()
            torch.cuda.synchronize()
            assert torch.equal(a, b), f"step {step}: graph replay differs from the eager step"
            for row, i in enumerate(order):
                live[i] = (live[i][0], int(a[row].argmax()))
    assert graphed.graph_replays + graphed.graph_captures == 24 and graphed.graph_captures >= len(graphed._graphs) >= 3 and graphed.graph_replays >= 12
    graphed.drop_graphs()


@pytest.mark.parametrize("name", ["b", "c"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_several_decode_steps_from_one_launch_equal_single_steps(folders, name, dtype):
    """decode_steps(): the device chooses each token, feeds it back in and moves the metadata on by
    itself.  Tokens and cache contents must equal those of single steps with the host in the loop,
    across page edges (page size 16, contexts from 3 to 70) and with fewer requests than the padded batch."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry

    folder, cfg, _ = folders[name]
    device = torch.device("cuda", 0)
    _, model = load_model(folder, dtype, device)
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (3, 30, 61)]

    def make():
        cache = CacheManager(model.cache_needs(), page_size=16, num_pages=40, max_requests=4, max_seq_len=256, dtype=dtype, device=device)
        return ModelRunner(model, cache, max_step_tokens=128, dtype=dtype, device=device, use_graph=True)

    single, several = make(), make()
    with torch.cuda.stream(torch.cuda.Stream(device)):
        state = []
        for runner in (single, several):
            caches, last = [], []
            for i, prompt in enumerate(prompts):
                caches.append(runner.cache.admit(i))
                last.append(int(runner.step([StepEntry(caches[-1], prompt, [len(prompt) - 1])])[0].argmax()))
            state.append((caches, last))
        assert state[0][1] == state[1][1]
        assert several.can_decode_steps([StepEntry(c, [t], [0]) for c, t in zip(*state[1])])
        want, got = [], []
        caches, last = state[0]
        for _ in range(9):
            logits = single.step([StepEntry(c, [t], [0]) for c, t in zip(caches, last)])
            last = logits.argmax(-1).tolist()
            want.append(last)
        caches, last = state[1]
        for steps in (4, 1, 4):
            chosen = several.decode_steps([StepEntry(c, [t], [0]) for c, t in zip(caches, last)], steps)
            assert len(chosen) == steps and all(len(row) == len(prompts) for row in chosen)
            got += chosen
            last = chosen[-1]
        torch.cuda.synchronize()
    assert got == want
    assert [c.length for c in state[0][0]] == [c.length for c in state[1][0]] == [len(p) + 9 for p in prompts]
    for a, b in zip(single.cache.layer_caches, several.cache.layer_caches):
        for request_a, request_b in zip(state[0][0], state[1][0]):
            pages_a, pages_b = request_a.tables[a.group], request_b.tables[b.group]
            assert torch.equal(a.k_pages[pages_a], b.k_pages[pages_b]) and torch.equal(a.v_pages[pages_a], b.v_pages[pages_b])
    several.drop_graphs()
    single.drop_graphs()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_step_on_another_stream_waits_for_the_work_that_built_the_runner(folders, dtype):
    """Weights are converted and cache pools cleared on the stream that is current when they are
    made; streams made by torch do not wait for that stream.  With the default stream kept busy
    while the model is bound and the runner built, the first step on a new stream must still see
    finished weights and cleared pools: its logits equal those of a run that waited for everything."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry

    folder, cfg, _ = folders["c"]
    device = torch.device("cuda", 0)
    prompt = np.random.default_rng(21).integers(0, cfg["vocab_size"], 90).tolist()
    busy = torch.randn(4096, 4096, device=device)
    results = []
    for wait_first in (True, False):
        if not wait_first:
            for _ in range(40):                 # tens of milliseconds of work ahead of the model's own
                busy = (busy @ busy).clamp_(-1, 1)
        _, model = load_model(folder, dtype, device)
        cache = CacheManager(model.cache_needs(), page_size=16, num_pages=12, max_requests=2, max_seq_len=128, dtype=dtype, device=device)
        runner = ModelRunner(model, cache, max_step_tokens=128, dtype=dtype, device=device)
        if wait_first:
            torch.cuda.synchronize()
        with torch.cuda.stream(torch.cuda.Stream(device)):
            entry = cache.admit(0)
            results.append(runner.step([StepEntry(entry, prompt, [0, len(prompt) - 1])]).float().cpu())
        torch.cuda.synchronize()
    assert torch.equal(results[0], results[1])


def test_seeded_sampling_is_reproducible_and_independent_of_batch_mates(folders):
    from llm_runtime_study_amd import Engine, SamplingConfig

    folder, cfg, _ = folders["b"]
    rng = np.random.default_rng(9)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (23, 40, 1, 64)]
    sampling = SamplingConfig(temperature=0.8, seed=0)
    engine = Engine.from_model_dir(folder, dtype="float32", max_seq_len=128, max_batch_size=4, max_num_batched_tokens=16)
    together = engine.generate_tokens(prompts, max_new_tokens=12, sampling=sampling, ignore_eos=True)
    again = engine.generate_tokens(prompts, max_new_tokens=12, sampling=sampling, ignore_eos=True)
    assert together == again and all(len(t) == 12 for t in together)
    alone = [engine.generate_tokens([p], max_new_tokens=12, sampling=sampling, ignore_eos=True)[0] for p in prompts]
    assert alone == together
    other = engine.generate_tokens(prompts, max_new_tokens=12, sampling=SamplingConfig(temperature=0.8, seed=1), ignore_eos=True)
    assert other != together
    greedy = engine.generate_tokens(prompts, max_new_tokens=12, ignore_eos=True)
    assert greedy != together
    top1 = engine.generate_tokens(prompts, max_new_tokens=12, sampling=SamplingConfig(temperature=0.8, top_k=1, seed=5), ignore_eos=True)
    assert top1 == greedy      # only the largest logit survives the filter


def test_graphs_of_large_batches_hold_library_products(folders):
    """More rows than the few-rows kernels take: the vendor library's matrix products are captured
    with the rest.  Every replay (24 of them, three padded sizes, eager prefill steps and
    synchronisations between them) must give the logits of the same step run eagerly."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry

    folder, cfg, _ = folders["c"]
    device, dtype = torch.device("cuda", 0), torch.bfloat16
    _, model = load_model(folder, dtype, device)
    rng = np.random.default_rng(31)

    def make(use_graph):
        cache = CacheManager(model.cache_needs(), page_size=16, num_pages=400, max_requests=64, max_seq_len=128, dtype=dtype, device=device)
        return ModelRunner(model, cache, max_step_tokens=256, dtype=dtype, device=device, use_graph=use_graph)

    eager, graphed = make(False), make(True)
    live = {}

    def admit(index):
        prompt = rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 40))).tolist()
        caches = (eager.cache.admit(index), graphed.cache.admit(index))
        a = eager.step([StepEntry(caches[0], prompt, [len(prompt) - 1])]).clone()
        b = graphed.step([StepEntry(caches[1], prompt, [len(prompt) - 1])]).clone()
        assert torch.equal(a, b)
        live[index] = (caches, int(a[0].argmax()))

    with torch.cuda.stream(torch.cuda.Stream(device)):
        for index in range(20):
            admit(index)
        for step in range(24):
            if step in (3, 4, 5, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20):     # 20 -> 35 requests: buckets 32 and 48
                admit(100 + step)
            if step == 22:                                                           # ... and down to 15: the own kernels' graphs
                for index in sorted(live)[:20]:
                    caches, _ = live.pop(index)
                    eager.cache.release(caches[0])
                    graphed.cache.release(caches[1])
            order = sorted(live)
            a = eager.step([StepEntry(live[i][0][0], [live[i][1]], [0]) for i in order]).clone()
            b = graphed.step([StepEntry(live[i][0][1], [live[i][1]], [0]) for i in order]).clone()
            torch.cuda.synchronize()
            assert torch.equal(a, b), f"step {step} with {len(order)} requests: graph replay differs from the eager step"
            for row, i in enumerate(order):
                live[i] = (live[i][0], int(a[row].argmax()))
    assert graphed.graph_replays + graphed.graph_captures == 24 and {key[0] for key in graphed._graphs} == {16, 32, 48}
    graphed.drop_graphs()


def test_graphs_of_up_to_128_rows_hold_this_packages_kernels(tmp_path):
    """A model whose matrices suit the kernel for 17..128 rows (every K a multiple of 256): batches of 40 to 100
    requests run as graphs of 48, 64, 96 and 128 rows of this package's kernels alone, and every replay gives the
    logits of the same step run eagerly, bit for bit; the logits agree with the float32 path."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.engine.loading import load_model
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry
    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.weights import write_model_dir

    raw = dict(TINY_C, vocab_size=352, hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2, head_dim=64)
    write_model_dir(config_from_dict(raw), seed=41, model_dir=tmp_path, init="scaled")
    device = torch.device("cuda", 0)
    _, model = load_model(tmp_path, torch.bfloat16, device)
    _, model32 = load_model(tmp_path, torch.float32, device)
    for n, k in ((4 * 64 + 2 * 2 * 64, 256), (256, 256), (1024, 256), (256, 512), (352, 256)):
        assert ops.gemm_mid_takes(torch.bfloat16, 100, n, k)
    rng = np.random.default_rng(32)

    def make(use_graph, m=model, dtype=torch.bfloat16):
        cache = CacheManager(m.cache_needs(), page_size=16, num_pages=500, max_requests=128, max_seq_len=96, dtype=dtype, device=device)
        return ModelRunner(m, cache, max_step_tokens=256, dtype=dtype, device=device, use_graph=use_graph, library_gemm=False)

    eager, graphed, exact = make(False), make(True), make(False, model32, torch.float32)
    live = {}

    def admit(index):
        prompt = rng.integers(0, raw["vocab_size"], int(rng.integers(2, 30))).tolist()
        caches = (eager.cache.admit(index), graphed.cache.admit(index), exact.cache.admit(index))
        a = eager.step([StepEntry(caches[0], prompt, [len(prompt) - 1])]).clone()
        b = graphed.step([StepEntry(caches[1], prompt, [len(prompt) - 1])]).clone()
        exact.step([StepEntry(caches[2], prompt, [])])
        assert torch.equal(a, b)
        live[index] = (caches, int(a[0].argmax()))

    with torch.cuda.stream(torch.cuda.Stream(device)):
        for index in range(40):
            admit(index)
        for step in range(12):
            for extra in range(6 if step < 10 else 0):                 # 40 -> 100 requests: buckets 48, 64, 96 and 128
                admit(1000 + step * 10 + extra)
            order = sorted(live)
            a = eager.step([StepEntry(live[i][0][0], [live[i][1]], [0]) for i in order]).clone()
            b = graphed.step([StepEntry(live[i][0][1], [live[i][1]], [0]) for i in order]).clone()
            c = exact.step([StepEntry(live[i][0][2], [live[i][1]], [0]) for i in order]).clone()
            torch.cuda.synchronize()
            assert torch.equal(a, b), f"step {step} with {len(order)} requests: graph replay differs from the eager step"
            error = (a - c).norm() / c.norm()
            assert error < 0.03, f"step {step}: bfloat16 logits are {float(error):.3f} of the float32 logits away"
            for row, i in enumerate(order):
                live[i] = (live[i][0], int(c[row].argmax()))
    assert graphed.graph_replays + graphed.graph_captures == 12 and {key[0] for key in graphed._graphs} == {48, 64, 96, 128}
    graphed.drop_graphs()


def test_sampled_tokens_do_not_depend_on_steps_per_launch(folders):
    """Seeded draws with top-k and top-p, one request greedy beside them: four decode steps from one
    launch (the device filters, draws and counts the draws itself) give the tokens of single steps."""
    from llm_runtime_study_amd import Engine, SamplingConfig

    folder, cfg, _ = folders["c"]
    rng = np.random.default_rng(21)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (9, 20, 4)]
    configs = [SamplingConfig(temperature=0.9, top_k=40, top_p=0.9, seed=5), SamplingConfig(),
               SamplingConfig(temperature=1.3, seed=77)]

    def run(per_launch):
        engine = Engine.from_model_dir(folder, dtype="bfloat16", max_seq_len=96, max_batch_size=3, decode_steps_per_launch=per_launch)
        scheduler = engine.create_scheduler(ignore_eos=True)
        for prompt, config in zip(prompts, configs):
            scheduler.add_request(prompt, max_new_tokens=11, sampling=config)
        tokens = {i: [] for i in range(len(prompts))}
        with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
            while scheduler.has_unfinished:
                for index, event in scheduler.step():
                    tokens[index].append(event.token_id)
        replays = engine.runner.graph_replays
        engine.runner.drop_graphs()
        return tokens, replays

    single, replays_single = run(1)
    several, replays_several = run(4)
    assert single == several and all(len(t) == 11 for t in single.values())
    assert len(set(single[0])) > 3 and len(set(single[2])) > 3        # draws, not a fixed point
    assert replays_several < replays_single


@pytest.mark.parametrize("graph,steps_per_launch", [(False, 1), (True, 1), (True, 4)], ids=["eager", "graph", "four-steps-a-launch"])
def test_logits_that_are_not_finite_abort_generation(folders, graph, steps_per_launch):
    """A request whose logits turn NaN while it decodes (the embedding row of its first generated token is
    poisoned) beside a healthy one: the step raises the reference's error (mini_llm/sampling.py:104-113), whether
    the host or the device chooses the tokens, every page comes back, and the engine generates again afterwards."""
    from llm_runtime_study_amd import Engine
    from llm_runtime_study_amd.errors import SamplingError

    folder, cfg, weights = folders["c"]
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (9, 14)]
    expected = [plain_greedy(cfg, weights, p, 6) for p in prompts]
    poisoned = expected[0][0]
    assert poisoned not in prompts[0] + prompts[1] + expected[1]
    engine = Engine.from_model_dir(folder, dtype="float32", max_seq_len=64, max_batch_size=2, max_num_batched_tokens=32,
                                   use_cuda_graph=graph, decode_steps_per_launch=steps_per_launch)
    assert engine.generate_tokens(prompts, max_new_tokens=6, ignore_eos=True) == expected
    row = engine.model.embedding[poisoned].clone()
    engine.model.embedding[poisoned] = float("nan")
    with pytest.raises(SamplingError, match="only finite values"):
        engine.generate_tokens(prompts, max_new_tokens=6, ignore_eos=True)
    manager = engine.cache_manager
    manager.check_invariants()
    assert manager.active_requests == 0 and manager.used_pages() == 0
    engine.model.embedding[poisoned] = row
    assert engine.generate_tokens(prompts, max_new_tokens=6, ignore_eos=True) == expected


def test_small_pool_makes_requests_wait_and_reuses_pages(folders):
    from llm_runtime_study_amd import Engine

    folder, cfg, weights = folders["a"]
    rng = np.random.default_rng(10)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (30, 25, 28, 12, 31, 5)]
    expected = [plain_greedy(cfg, weights, p, 6, [cfg["eos_token_id"]]) for p in prompts]
    # 6 pages of 16 tokens: two requests of up to 37 tokens (3 pages each) at a time
    engine = Engine.from_model_dir(folder, dtype="float32", max_seq_len=48, max_batch_size=4, num_pages=6, max_num_batched_tokens=24)
    scheduler = engine.create_scheduler()
    for p in prompts:
        scheduler.add_request(p, max_new_tokens=6)
    got = {i: [] for i in range(len(prompts))}
    most_running, waited_for_pages = 0, False
    with torch.cuda.stream(engine.stream):
        while scheduler.has_unfinished:
            for i, e in scheduler.step():
                got[i].append(e.token_id)
            most_running = max(most_running, scheduler.num_running)
            waited_for_pages |= scheduler.num_waiting > 0 and scheduler.num_running < 4
            engine.cache_manager.check_invariants()
            assert engine.cache_manager.tables_match_device()
    assert [got[i] for i in range(len(prompts))] == expected
    assert 2 <= most_running <= 3 and waited_for_pages and engine.cache_manager.used_pages() == 0


@pytest.mark.parametrize("steps_per_launch,ahead,ends", [(1, False, False), (4, False, False), (4, True, False), (4, True, True)],
                         ids=["one-step", "four-steps", "four-steps-queued-ahead", "queued-ahead-with-ends-of-sequence"])
def test_many_requests_through_the_scheduler_equal_each_alone(steps_per_launch, ahead, ends):
    """Forty requests of random lengths, two in three greedy and the others with seeded top-k / top-p
    sampling, arriving a few at a time into continuous batching with portions of at most 48 tokens, a
    pool of 40 pages and up to eight running: in float32 every request's tokens are exactly those it
    produces alone, and the pool is empty at the end.  ends: a tenth of the vocabulary ends a sequence, so
    requests end inside launches while the launch after is already queued."""
    from llm_runtime_study_amd import Engine, SamplingConfig
    from llm_runtime_study_amd.config import config_from_dict

    cfg = config_from_dict(dict(TINY_C, eos_token_id=list(range(0, TINY_C["vocab_size"], 10))) if ends else TINY_C)
    rng = np.random.default_rng(5)
    requests = []
    for i in range(40):
        prompt = rng.integers(0, cfg.vocab_size, int(rng.integers(1, 120))).tolist()
        sampling = SamplingConfig() if i % 3 else SamplingConfig(temperature=0.8, top_k=20, top_p=0.9, seed=i)
        requests.append((prompt, int(rng.integers(1, 40 if not ends else 90)), sampling))
    alone = Engine.from_config(cfg, seed=1, init="scaled", dtype="float32", max_seq_len=256, max_batch_size=1, decode_steps_per_launch=1, launch_ahead=False)
    want = [alone.generate_tokens([p], max_new_tokens=n, sampling=s, ignore_eos=not ends)[0] for p, n, s in requests]
    if ends:
        assert sum(len(w) < n for w, (_, n, _) in zip(want, requests)) >= 10     # many do end early
    engine = Engine.from_config(cfg, seed=1, init="scaled", dtype="float32", max_seq_len=256, max_batch_size=8,
                                max_num_batched_tokens=48, num_pages=40, decode_steps_per_launch=steps_per_launch, launch_ahead=ahead)
    scheduler = engine.create_scheduler(ignore_eos=not ends)
    got, pending = {}, list(requests)
    with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
        while pending or scheduler.has_unfinished:
            for _ in range(int(rng.integers(0, 3))):
                if pending:
                    prompt, n, sampling = pending.pop(0)
                    got[scheduler.add_request(prompt, max_new_tokens=n, sampling=sampling)] = []
            if scheduler.has_unfinished:
                for index, event in scheduler.step():
                    got[index].append(event.token_id)
                engine.cache_manager.check_invariants()
                assert engine.cache_manager.tables_match_device()
    assert [got[i] for i in range(len(requests))] == want
    assert engine.cache_manager.used_pages() == 0


def test_engine_changes_precision_and_hands_out_caches(folders):
    """Engine.to(dtype=...) makes the weights again in the other precision (float32 after bfloat16 is
    the checkpoint's precision, not a widened bfloat16) and refuses while a cache is out;
    allocate_cache / release_cache are the reference's calls for driving the step function by hand."""
    from llm_runtime_study_amd import Engine
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.errors import EngineError

    folder, cfg, weights = folders["b"]
    prompt = [5, 9, 200, 31, 7, 7, 120]
    expected = plain_greedy(cfg, weights, prompt, 8, [cfg["eos_token_id"]])
    engine = Engine.from_model_dir(folder, dtype="bfloat16", max_seq_len=64, max_batch_size=2)
    first = engine.generate_tokens([prompt], max_new_tokens=8)[0]
    assert sum(a == b for a, b in zip(first, expected)) >= 6
    assert engine.to(dtype="bfloat16") is engine
    engine.to(dtype="float32")
    assert engine.dtype == torch.float32 and engine.cache_manager.dtype == torch.float32
    assert engine.generate_tokens([prompt], max_new_tokens=8)[0] == expected
    cache = engine.allocate_cache(32)
    with pytest.raises(EngineError, match="while request caches are active"):
        engine.to(dtype="bfloat16")
    with torch.cuda.stream(engine.stream):
        logits = engine.runner.step([StepEntry(cache, prompt, [len(prompt) - 1])])
        assert int(logits[0].argmax()) == expected[0]
    engine.release_cache(cache)
    engine.release_cache(cache)
    assert engine.cache_manager.used_pages() == 0
    with pytest.raises(EngineError, match="capacity"):
        engine.allocate_cache(65)
    with pytest.raises(EngineError, match="runs on the GPU only"):
        engine.to(device="cpu")
    engine.to(dtype="bfloat16")
    assert engine.generate_tokens([prompt], max_new_tokens=8)[0] == first


def test_command_line_on_the_gpu(folders):
    folder, cfg, weights = folders["a"]
    expected = plain_greedy(cfg, weights, [5, 6, 7], 4, [cfg["eos_token_id"]])
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt-ids", "5,6,7",
                           "--max-new-tokens", "4", "--max-seq-len", "64", "--dtype", "float32"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[0].split() == [str(t) for t in expected]
    assert "prompt tokens:       3" in proc.stdout and "stop reason:" in proc.stdout
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt", "hello", "--max-seq-len", "64"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 2 and "error: a text prompt needs a tokenizer" in proc.stderr
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt-ids", "1", "--max-seq-len", "4096"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 2 and "exceeds the model limit" in proc.stderr


@pytest.mark.gpu
def test_staggered_benchmark_runs_every_request_to_its_limit(capsys):
    """The staggered serving run on one layer of the 8B shape: six requests, a pool for four, portions of
    32 tokens; every request produces exactly its output limit and the report holds the reference's figures."""
    import json

    from llm_runtime_study_amd.benchmarks import staggered

    code = staggered.main(["--shape", "8b", "--layers", "1", "--requests", "6", "--interval-ms", "1", "--prompt-tokens", "16,64",
                           "--new-tokens", "4,8", "--max-batch-size", "4", "--step-tokens", "32", "--max-seq-len", "128",
                           "--warmups", "0", "--seed", "1"])
    assert code == 0
    report = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    import numpy as np
    drawn = staggered.draw_requests(np.random.default_rng(1), 151936, 6, (16, 64), (4, 8))
    assert report["generated_tokens"] == sum(n for _, n in drawn)
    assert report["prompt_tokens"] == sum(len(p) for p, _ in drawn)
    assert report["makespan_s"] > 0 and report["output_tok_s"] > 0
    assert 0 < report["ttft_ms_p50"] <= report["ttft_ms_p95"] <= report["latency_ms_p95"]
    assert report["latency_ms_p50"] <= report["latency_ms_p95"] <= 1000.0 * report["makespan_s"] + 1e-6


@pytest.mark.gpu
def test_host_cost_benchmark_times_the_three_ways_of_launching_a_step(capsys):
    """One layer of the 8B shape, a 64-token portion beside two decoding requests: the report holds the three
    ways of launching, the plan is recorded once and replayed for every timed step, and every timed step of the
    third way is a launch of the plan's graph."""
    import json

    from llm_runtime_study_amd.benchmarks import host_cost

    code = host_cost.main(["--shape", "8b", "--layers", "1", "--tokens", "64", "--decoding", "2", "--context", "40", "--repeats", "3"])
    assert code == 0
    report = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    for way in ("through_parts", "from_plan", "from_graph_of_plan"):
        assert 0 < report[way]["host_ms"] <= report[way]["total_ms"]
    assert report["from_plan"]["replays"] >= 3 and report["from_graph_of_plan"]["replays"] >= 3
    # two shapes are recorded, once each: the step that reads a decoding request's context and the timed step
    assert report["from_plan"]["recordings"] == 2 and report["from_graph_of_plan"]["recordings"] == 2
    assert report["from_graph_of_plan"]["graph_replays"] >= 3


def test_a_cache_pool_the_device_cannot_hold_is_refused_before_anything_is_allocated():
    """64 requests of 1,048,576 tokens for 36 layers of 8 kv heads of 128: 9 TiB of pages.  The error says what
    was asked for, what is free and what would fit; nothing was allocated."""
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.parts import PagedKVNeed
    from llm_runtime_study_amd.errors import KVCacheError

    before = torch.cuda.memory_allocated()
    with pytest.raises(KVCacheError, match=r"needs 9\d\d\d\.\d GiB.*GiB are free.*would fit"):
        CacheManager([PagedKVNeed(8, 128, None)] * 36, page_size=16, num_pages=64 * 65536, max_requests=64, max_seq_len=1 << 20,
                     dtype=torch.bfloat16, device="cuda")
    assert torch.cuda.memory_allocated() == before


def test_one_segment_of_device_memory_is_reserved_for_an_engine_and_its_tensors_come_out_of_it(folders):
    """engine/loading.py: the reservation is one allocation that torch's allocator keeps; what is allocated next is
    cut out of it (torch asks the device for nothing more); an engine too small to gain reserves nothing, a size the
    device does not have is no error, and the option switches it off."""
    from llm_runtime_study_amd import Engine
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine import loading
    from llm_runtime_study_amd.models import DecoderModel

    tiny = config_from_dict(TINY_B)
    model = DecoderModel(spec_for(tiny))
    weights = sum(int(np.prod(spec.shape)) for spec in model.tensors().values())
    pages = 2 * TINY_B["num_key_value_heads"] * TINY_B["head_dim"] * TINY_B["num_hidden_layers"] * 16 * (40 + 1)
    assert loading.engine_bytes(model, torch.bfloat16, 16, 40) == 2 * (weights + pages)
    assert loading.engine_bytes(model, torch.float32, 16, 40) == 4 * (weights + pages)
    assert loading.reserve_for(tiny, torch.bfloat16, "cuda", 16, 40) == 0          # far under a gigabyte
    assert loading.reserve_device_memory(1 << 50, "cuda") == 0                     # a petabyte: refused, nothing raised
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_reserved()
    got = loading.reserve_device_memory(1 << 30, "cuda")
    assert got == 3 << 30 and torch.cuda.memory_reserved() == before + got         # a gigabyte and the margin, in whole gigabytes
    first = torch.empty(700 << 20, dtype=torch.uint8, device="cuda")
    second = torch.empty(900 << 20, dtype=torch.uint8, device="cuda")
    assert torch.cuda.memory_reserved() == before + got                            # both were cut out of what torch holds
    del first, second
    torch.cuda.empty_cache()
    assert torch.cuda.memory_reserved() == before
    folder = folders["b"][0]
    engine = Engine.from_model_dir(folder, max_seq_len=128, max_batch_size=2, reserve_memory=False)
    assert engine.generate_tokens([[5, 6, 7]], max_new_tokens=3) == Engine.from_model_dir(
        folder, max_seq_len=128, max_batch_size=2).generate_tokens([[5, 6, 7]], max_new_tokens=3)
