"""Replays the same requests under every way of cutting them and compares each logits row
with the plain whole-sequence implementation: alone and whole; most in one step and the
last 32 tokens one by one; portions of changing size down to two tokens; and mixed, up to
four live requests with so few pages that they are used again.  float32 and bfloat16."""

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
LENGTHS = {"a": [5, 11, 17, 64, 65, 127, 33, 90], "b": [1, 23, 40, 64, 200, 331, 129, 77, 16], "c": [2, 34, 64, 130, 300, 95, 600],
           "d": [3, 48, 64, 129, 270, 31, 500, 18], "e": [4, 30, 64, 101, 77, 50, 120, 9]}
# heads of 128 dims (the size whose attention kernel for ragged steps is another one, and prepares the queries itself), three
# query heads to a kv head (one wave of the kernel's four has none); the other sizes small
# a large eps (0.3, where the others have 1e-5 and less): a norm that took another eps than the configuration's, such as
# the per-head norms of q and k with a constant of their own, would show in every row
TINY_E = dict(TINY_A, rms_norm_eps=0.3, vocab_size=211, num_attention_heads=6, num_key_value_heads=3, head_dim=32, hidden_size=72)
TINY_D = dict(TINY_C, head_dim=128, num_attention_heads=6, num_key_value_heads=2, vocab_size=290, hidden_size=96, intermediate_size=144)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """Model folders of the tiny configurations, their requests and the plain logits."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    out = {}
    for name, raw in (("a", TINY_A), ("b", TINY_B), ("c", TINY_C), ("d", TINY_D), ("e", TINY_E)):
        folder = tmp_path_factory.mktemp(f"model_{name}")
        write_model_dir(config_from_dict(raw), seed={"a": 11, "b": 12, "c": 13, "d": 14, "e": 15}[name], model_dir=folder, init="scaled")
        cfg, weights = plain.load_model_dir(folder, torch.float64)
        rng = np.random.default_rng(5)
        requests = {f"{name}{i}": rng.integers(0, raw["vocab_size"], n).tolist() for i, n in enumerate(LENGTHS[name])}
        want = {key: plain.qwen3_forward(weights, cfg, toks) for key, toks in requests.items()}
        out[name] = (folder, raw, requests, want)
    return out


def run_replay(folder, dtype, steps, max_tokens, tmp_path, page_size=16, as_the_engine=False, counters=None):
    """as_the_engine: on a stream of its own with graphs on, as Engine runs its steps: decode-only steps are graph
    replays, and step shapes that come back are launched as the graph of their recorded plan."""
    from llm_runtime_study_amd.engine import trace

    out_dir = tmp_path / "logits"
    if as_the_engine:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            runner = trace.make_runner(folder, dtype, max_tokens, page_size, use_graph=True)
            trace.replay(runner, traces.strip(steps).splitlines(), out_dir, echo=lambda _: None)
            side.synchronize()
        if counters is not None:
            counters.update(graph_replays=runner.graph_replays, plan_replays=runner.plan_replays, plan_graph_replays=runner.plan_graph_replays)
        runner.drop_graphs()
    else:
        runner = trace.make_runner(folder, dtype, max_tokens, page_size)
        trace.replay(runner, traces.strip(steps).splitlines(), out_dir, echo=lambda _: None)
    runner.cache.check_invariants()
    assert runner.cache.active_requests == 0 and runner.cache.used_pages() == 0
    assert runner.cache.tables_match_device()
    return out_dir


def compare(got, want, dtype):
    """Every row that was asked for, against the plain logits of the same position.  bfloat16: the row as a whole
    (relative L2), and its first choice: the token the engine rates highest is the plain implementation's, or one
    that the plain implementation rates within 6 % of its largest logit of the best (a single logit far off, which
    the norm of 300 would hide, fails this), and nine rows in ten agree outright."""
    checked = agree = 0
    for key, rows in got.items():
        for position, row in rows.items():
            ref = want[key][position]
            if dtype == "float32":
                torch.testing.assert_close(row.double(), ref, rtol=1e-4, atol=1e-4, msg=lambda m: f"{key}@{position}: {m}")
                assert int(row.argmax()) == int(ref.argmax()) or ref.topk(2).values.diff().abs() < 2e-4, f"{key}@{position}: first choice differs"
            else:
                err = (row.double() - ref).norm() / ref.norm()
                assert err < 3e-2, f"{key}@{position}: relative error {err:.3g}"
                mine, best = int(row.argmax()), int(ref.argmax())
                agree += mine == best
                assert ref[best] - ref[mine] <= 6e-2 * ref.abs().max(), f"{key}@{position}: first choice {mine} is rated {ref[mine]:.3f}, the plain one {best} {ref[best]:.3f}"
            checked += 1
    if dtype != "float32" and checked:
        assert agree >= 0.9 * checked, f"first choices agree in {agree} of {checked} rows"
    return checked


def round64(n):
    return -(-n // 64) * 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
def test_whole(models, name, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    steps = traces.whole(requests)
    out = run_replay(folder, dtype, steps, max(round64(len(t)) for t in requests.values()), tmp_path)
    got = traces.collect(steps, out, raw["vocab_size"])
    assert compare(got, want, dtype) == sum(len(t) for t in requests.values())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
def test_prefill_then_last_32_one_by_one(models, name, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    steps = traces.prefill_then_decode(requests, tail=32)
    out = run_replay(folder, dtype, steps, max(round64(len(t)) for t in requests.values()), tmp_path)
    compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("a", 16), ("b", 16), ("b", 4), ("a", 64), ("c", 32), ("d", 16), ("d", 64)])
def test_portions_of_changing_size(models, name, page, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    steps = traces.portions(requests)
    out = run_replay(folder, dtype, steps, max(round64(len(t)) for t in requests.values()), tmp_path, page)
    compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("a", 0), ("b", 1), ("b", 2), ("c", 3), ("d", 4), ("d", 5), ("e", 6)])
def test_mixed_with_reused_pages(models, name, seed, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    budget = 2 * max(round64(len(t)) for t in requests.values())
    steps, peak = traces.mixed(requests, seed=seed, max_live=4, max_tokens=budget)
    assert max(len(s["entries"]) for s in steps) >= 3
    out = run_replay(folder, dtype, steps, peak, tmp_path)
    got = traces.collect(steps, out, raw["vocab_size"])
    assert compare(got, want, dtype) > 50
    # the pool was smaller than what all requests together need: pages were used again
    assert peak < sum(round64(len(t)) for t in requests.values())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_the_four_ways_on_the_engines_path_of_graphs(models, name, dtype, tmp_path):
    """The same four replays on a stream of the runner's own with graphs on, which is how Engine runs: single-token
    steps are replays of decode graphs, shapes that come back are launched from the graph of their recorded plan.
    Every row against the plain implementation, as on the eager path."""
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    seen = {}
    steps = traces.whole(requests)
    out = run_replay(folder, dtype, steps, longest, tmp_path / "whole", as_the_engine=True)
    assert compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype) == sum(len(t) for t in requests.values())
    steps = traces.prefill_then_decode(requests, tail=32)
    out = run_replay(folder, dtype, steps, longest, tmp_path / "tail", as_the_engine=True, counters=seen)
    compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype)
    assert seen["graph_replays"] >= 20 * len(requests)             # the single tokens ran as graphs
    steps = traces.portions(requests)
    out = run_replay(folder, dtype, steps, longest, tmp_path / "portions", as_the_engine=True, counters=seen)
    compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype)
    assert seen["plan_graph_replays"] >= 10                        # portions of one size came back: graphs of plans
    steps, peak = traces.mixed(requests, seed=7, max_live=4, max_tokens=2 * longest)
    out = run_replay(folder, dtype, steps, peak, tmp_path / "mixed", as_the_engine=True, counters=seen)
    assert compare(traces.collect(steps, out, raw["vocab_size"]), want, dtype) > 50
    assert seen["graph_replays"] + seen["plan_replays"] > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_late_portions_and_single_tokens_of_a_long_prompt(tmp_path, dtype):
    """2,300 tokens: most in one step, then portions of 40, 16, 2 and 1 tokens and a step that holds a
    portion of this request beside a single token of another.  With so few queries over more than a
    thousand keys the bfloat16 attention kernel divides each group's keys between workgroups."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    raw = dict(TINY_C, max_position_embeddings=4096)
    folder = tmp_path / "model"
    write_model_dir(config_from_dict(raw), seed=14, model_dir=folder, init="scaled")
    cfg, weights = plain.load_model_dir(folder, torch.float64)
    rng = np.random.default_rng(9)
    long_ids = rng.integers(0, raw["vocab_size"], 2300).tolist()
    other = rng.integers(0, raw["vocab_size"], 1200).tolist()
    want = {"long": plain.qwen3_forward(weights, cfg, long_ids), "other": plain.qwen3_forward(weights, cfg, other)}
    steps, at = [], 0
    cuts = [2200, 40, 16, 2, 1, 30, 11]
    for number, n in enumerate(cuts):
        entries = [{"id": "long", "tokens": long_ids[at:at + n], "want": list(range(max(0, n - 48), n))}]
        if number == 0:
            entries.append({"id": "other", "tokens": other[:1199], "want": [1198]})
        if number == 5:     # a single token of the other request beside a portion of this one
            entries.insert(0, {"id": "other", "tokens": other[1199:], "want": [0]})
        steps.append({"step": number, "entries": entries, "end": ["long", "other"] if number == len(cuts) - 1 else []})
        at += n
    assert at == len(long_ids)
    out = run_replay(folder, dtype, steps, 2304 + 1216, tmp_path)
    got = traces.collect(steps, out, raw["vocab_size"])
    assert compare(got, want, dtype) == 48 + 40 + 16 + 2 + 1 + 30 + 11 + 2


def test_cuts_agree_bit_for_bit_in_float32(models, tmp_path):
    """In float32 the order of every sum depends on the position alone, so whole, portioned and
    mixed replays give identical bits."""
    folder, raw, requests, _ = models["b"]
    a = traces.whole(requests)
    b = traces.portions(requests)
    ga = traces.collect(a, run_replay(folder, "float32", a, 384, tmp_path / "w"), raw["vocab_size"])
    gb = traces.collect(b, run_replay(folder, "float32", b, 384, tmp_path / "p"), raw["vocab_size"])
    for key in ga:
        for position in ga[key]:
            assert torch.equal(ga[key][position], gb[key][position]), f"{key}@{position}"


def test_trace_run_program(models, tmp_path):
    """The program itself: reads steps on stdin, prints `done <step>` after each, exits 0."""
    folder, raw, requests, want = models["a"]
    few = dict(list(requests.items())[:3])
    steps, peak = traces.mixed(few, seed=3, max_live=3)
    out = tmp_path / "o"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
         "--out", str(out), "--max-tokens", str(peak)],
        input=traces.strip(steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    done = [line for line in proc.stdout.splitlines() if line.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps]
    compare(traces.collect(steps, out, raw["vocab_size"]), want, "float32")
