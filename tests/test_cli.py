"""Command line: options, streaming, metrics and error exit code, with a fake engine (CPU)."""

import io
from types import SimpleNamespace

import pytest

from llm_runtime_study_amd import cli
from llm_runtime_study_amd.engine.scheduler import GenerationEvent
from llm_runtime_study_amd.errors import ConfigError
from llm_runtime_study_amd.sampling import SamplingConfig
from llm_runtime_study_amd.errors import SamplingError


def test_parser_has_the_reference_options_and_defaults():
    # reference mini_llm/cli.py:32-64
    args = cli.build_parser().parse_args(["--model", "m", "--prompt", "hi"])
    assert (args.max_new_tokens, args.max_seq_len, args.temperature, args.top_k, args.top_p, args.seed) == (128, 4096, 0.0, None, 1.0, None)
    assert (args.device, args.dtype, args.interactive, args.thinking, args.no_stream, args.no_metrics) == ("auto", "auto", False, False, False, False)
    assert args.random_weights is None and cli.build_parser().parse_args(["--model", "m", "--random-weights", "7", "--device", "hip"]).random_weights == 7
    with pytest.raises(SystemExit):
        cli.build_parser().parse_args(["--prompt", "hi"])


def fake_engine(events):
    calls = {}

    def generate(prompts, **options):
        calls["prompts"], calls["options"] = prompts, options
        return iter([(0, e) for e in events])

    return SimpleNamespace(generate=generate, tokenizer=object(), device="cuda:0", dtype="torch.bfloat16", load_seconds=1.5,
                           last_cache_capacity=48, last_cache_num_bytes=48 * 1024), calls


def test_streams_text_and_prints_metrics(monkeypatch):
    events = [GenerationEvent(5, 0, "Hel", "Hel", None, 0.5, 7), GenerationEvent(6, 1, "lo", "Hello", "max_new_tokens", 0.25, None)]
    engine, calls = fake_engine(events)
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    out = io.StringIO()
    code = cli.main(["--model", "m", "--prompt", "hi", "--max-new-tokens", "2", "--temperature", "0.7", "--top-k", "5", "--seed", "3"], output=out)
    text = out.getvalue()
    assert code == 0 and text.startswith("Hello\n")
    assert "prompt tokens:       7" in text and "generated tokens:    2" in text and "stop reason:         max_new_tokens" in text
    assert "decode throughput:   4.00 tokens/s" in text and "(48 positions)" in text
    assert calls["options"]["sampling"] == SamplingConfig(temperature=0.7, top_k=5, top_p=1.0, seed=3)
    assert calls["options"]["max_new_tokens"] == 2 and calls["prompts"][0][0].content == "hi"


def test_prompt_ids_and_no_stream(monkeypatch):
    engine, calls = fake_engine([GenerationEvent(9, 0, "", "", "eos", None, 3)])
    engine.tokenizer = None
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    out = io.StringIO()
    assert cli.main(["--model", "m", "--prompt-ids", "4, 5,6", "--no-stream", "--no-metrics"], output=out) == 0
    assert calls["prompts"][0] == [4, 5, 6] and out.getvalue() == "9\n"


def test_typed_errors_exit_with_2(monkeypatch):
    def boom(args):
        raise ConfigError("model directory does not exist: m")

    monkeypatch.setattr(cli, "open_engine", boom)
    err = io.StringIO()
    assert cli.main(["--model", "m", "--prompt", "hi"], error=err) == 2
    assert err.getvalue() == "error: model directory does not exist: m\n"
    err = io.StringIO()
    assert cli.main(["--model", "m"], error=err) == 2 and "--prompt is required" in err.getvalue()
    err = io.StringIO()
    assert cli.main(["--model", "m", "--prompt", "x", "--temperature", "-1"], error=err) == 2 and "temperature" in err.getvalue()


def test_metrics_block_has_the_reference_layout(monkeypatch):
    """Every line of the block as the reference prints it (mini_llm/cli.py:213-247): two spaces, the name with
    its colon padded to 21 columns, the value."""
    events = [GenerationEvent(5, 0, "a", "a", None, 0.5, 3), GenerationEvent(6, 1, "b", "ab", None, 0.5, None),
              GenerationEvent(7, 2, "c", "abc", "eos", 0.5, None)]
    engine, _ = fake_engine(events)
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    out = io.StringIO()
    assert cli.main(["--model", "m", "--prompt", "hi"], output=out) == 0
    lines = out.getvalue().split("\n")
    assert lines[:3] == ["abc", "", "metrics"]
    assert lines[3:6] == ["  device:              cuda:0", "  dtype:               torch.bfloat16", "  load time:           1.50 s"]
    assert lines[6:9] == ["  prompt tokens:       3", "  generated tokens:    3", "  cache:               0.05 MiB (48 positions)"]
    assert lines[9].startswith("  time to first token: ") and lines[9].endswith(" ms")
    assert lines[10:12] == ["  decode throughput:   2.00 tokens/s", "  stop reason:         eos"]


def test_an_answer_without_events_or_without_a_prompt_count_is_an_error(monkeypatch):
    engine, _ = fake_engine([])
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    err = io.StringIO()
    assert cli.main(["--model", "m", "--prompt", "hi"], output=io.StringIO(), error=err) == 2 and "without a terminal event" in err.getvalue()
    engine, _ = fake_engine([GenerationEvent(5, 0, "a", "a", "eos", 0.5, None)])
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    err = io.StringIO()
    assert cli.main(["--model", "m", "--prompt", "hi"], output=io.StringIO(), error=err) == 2 and "prompt-token count" in err.getvalue()
    err = io.StringIO()
    assert cli.main(["--model", "m", "--prompt-ids", "4,x"], output=io.StringIO(), error=err) == 2 and "comma-separated integers" in err.getvalue()


def test_interactive_goes_on_after_a_failed_prompt(monkeypatch):
    from llm_runtime_study_amd.errors import GenerationError

    answers = iter([GenerationError("prompt has 9 tokens but model context limit is 4"), [GenerationEvent(5, 0, "fine", "fine", "eos", None, 2)]])

    def generate(prompts, **options):
        item = next(answers)
        if isinstance(item, Exception):
            raise item
        return iter([(0, e) for e in item])

    engine, _ = fake_engine([])
    engine.generate = generate
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    out, err = io.StringIO(), io.StringIO()
    code = cli.main(["--model", "m", "--interactive", "--no-metrics", "--prompt", "first"], input_stream=io.StringIO("second\n"), output=out, error=err)
    assert code == 0 and err.getvalue() == "error: prompt has 9 tokens but model context limit is 4\n"
    assert "you> first" in out.getvalue() and "assistant> fine" in out.getvalue()


def test_sampling_config_validation():
    # reference tests/test_generation.py:69-80
    for bad in (dict(temperature=-1), dict(top_k=0), dict(top_p=0), dict(top_p=1.5), dict(seed=-1), dict(temperature=float("nan"))):
        with pytest.raises(SamplingError):
            SamplingConfig(**bad)
    assert SamplingConfig().greedy and not SamplingConfig(temperature=0.3).greedy


def test_interactive_reads_until_quit(monkeypatch):
    engine, calls = fake_engine([GenerationEvent(5, 0, "ok", "ok", "eos", None, 2)])
    monkeypatch.setattr(cli, "open_engine", lambda args: engine)
    out = io.StringIO()
    code = cli.main(["--model", "m", "--interactive", "--no-metrics"], input_stream=io.StringIO("hello\n\n/quit\n"), output=out)
    assert code == 0 and "assistant> ok" in out.getvalue() and out.getvalue().count("you> ") == 3


def test_bench_refuses_more_than_one_gpu_with_one_line_and_exit_code_2():
    """The benchmark's contract: this engine runs on one GPU; asked for more it says so in one line."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    proc = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    lines = [line for line in proc.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bench_counts_the_flops_and_the_lead_of_early_requests():
    import bench

    from llm_runtime_study_amd.config import config_from_dict

    from llm_runtime_study_amd.config import spec_for
    from llm_runtime_study_amd.models import DecoderModel

    # the model says its own operations, part by part, from the tensors it declares (nothing is allocated for that)
    model = DecoderModel(spec_for(config_from_dict(bench.QWEN3_8B)))
    per_layer = (32 + 16) * 128 * 4096 + 4096 * 4096 + 3 * 4096 * 12288
    linear = 2.0 * 2048 * per_layer * 36 + 2.0 * 4096 * 151936
    attention = 4.0 * (2048 * 2049 / 2) * 32 * 128 * 36
    assert bench.prefill_flops(model, 2048) == linear + attention
    assert model.flops(8, 8 * 2049, 8) == 2.0 * 8 * per_layer * 36 + 8 * 2.0 * 4096 * 151936 + 4.0 * 8 * 2049 * 32 * 128 * 36
    # eight prompts of 2,048 tokens read one a step: the first request is seven tokens ahead of the last
    assert bench.decode_lead(8, 2048, 2048) == 7
    assert bench.decode_lead(8, 32768, 2048) == 7 * 16 and bench.decode_lead(1, 5000, 2048) == 0
    assert set(bench.SHAPES) == {"0.6b", "1.7b", "4b", "8b", "14b", "32b"} and bench.SHAPES["32b"]["num_hidden_layers"] == 64


def test_staggered_benchmark_percentiles_and_drawn_requests():
    """Nearest-rank percentiles as the reference takes them (benchmarks/common.py:91-95); the same
    seed draws the same requests, inside the asked ranges."""
    import numpy as np

    from llm_runtime_study_amd.benchmarks import staggered

    assert staggered.percentile([4.0, 1.0, 3.0, 2.0], 0.5) == 2.0
    assert staggered.percentile([4.0, 1.0, 3.0, 2.0], 0.95) == 4.0
    assert staggered.percentile([7.0], 0.95) == 7.0
    assert staggered.span("128,2048") == (128, 2048) and staggered.span("64") == (64, 64)
    first = staggered.draw_requests(np.random.default_rng(3), 331, 20, (5, 9), (2, 4))
    again = staggered.draw_requests(np.random.default_rng(3), 331, 20, (5, 9), (2, 4))
    assert first == again
    assert all(5 <= len(p) <= 9 and 2 <= n <= 4 and all(0 <= t < 331 for t in p) for p, n in first)
    assert {len(p) for p, _ in first} == {5, 6, 7, 8, 9}
