"""Staggered-arrival serving run: continuous batching with chunked prefill, random weights.

    python -m llm_runtime_study_amd.benchmarks.staggered [--shape 14b] [--requests 64] [--interval-ms 50]
        [--prompt-tokens 128,2048] [--new-tokens 128,512] [--max-batch-size 64] [--step-tokens 512]
        [--max-seq-len 4096] [--layers L] [--repeats 1] [--seed 0]

Requests arrive `interval` apart on the wall clock (0: all at once); prompt lengths and output limits
are drawn uniformly from the given ranges with the seed, token ids uniformly from the vocabulary (no
text, no dataset).  Requests run to their output limit (random weights never mean an end-of-sequence
token).  It reports what the reference's staggered benchmark reports (benchmarks/staggered.py:17-30,
176-199): makespan, output tokens a second, and the p50 / p95 of the time to the first token and of
the request latency, counted from each request's arrival; one JSON line.
"""

from __future__ import annotations

import argparse
import json
import math
import statistics
import sys
import time

from .shapes import SHAPES


def percentile(values, fraction: float) -> float:
    """Nearest-rank percentile, as the reference takes it (benchmarks/common.py:91-95)."""
    ordered = sorted(values)
    if not ordered:
        raise ValueError("percentile of nothing")
    return ordered[max(0, math.ceil(fraction * len(ordered)) - 1)]


def span(text: str) -> tuple[int, int]:
    parts = [int(p) for p in text.split(",")]
    if len(parts) == 1:
        parts = parts * 2
    if len(parts) != 2 or parts[0] <= 0 or parts[1] < parts[0]:
        raise argparse.ArgumentTypeError(f"expected LOW,HIGH with 0 < LOW <= HIGH, got {text!r}")
    return parts[0], parts[1]


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="staggered", description=__doc__.splitlines()[0])
    parser.add_argument("--shape", choices=tuple(SHAPES), default="14b")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (reported)")
    parser.add_argument("--requests", type=int, default=64)
    parser.add_argument("--interval-ms", type=float, default=50.0)
    parser.add_argument("--prompt-tokens", type=span, default=(128, 2048))
    parser.add_argument("--new-tokens", type=span, default=(128, 512))
    parser.add_argument("--max-batch-size", type=int, default=64)
    parser.add_argument("--step-tokens", type=int, default=512, help="token budget of a step (portions of prompts beside decoded tokens)")
    parser.add_argument("--max-seq-len", type=int, default=4096)
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--repeats", type=int, default=1)
    parser.add_argument("--warmups", type=int, default=1, help="whole untimed runs before the timed ones (they also capture the decode graphs)")
    parser.add_argument("--seed", type=int, default=0)
    return parser


def draw_requests(rng, vocab: int, count: int, prompt_span, new_span):
    return [(rng.integers(0, vocab, int(rng.integers(prompt_span[0], prompt_span[1] + 1))).tolist(),
             int(rng.integers(new_span[0], new_span[1] + 1))) for _ in range(count)]


def run_once(engine, requests, interval: float) -> dict:
    """One replay.  Times are seconds from the first arrival."""
    import torch

    from ..sampling import SamplingConfig

    scheduler = engine.create_scheduler(ignore_eos=True)
    arrivals = [i * interval for i in range(len(requests))]
    first, finish = {}, {}
    generated = 0
    steps = 0
    submitted = 0
    index_of = {}
    with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
        engine.synchronize()
        start = time.perf_counter()
        while submitted < len(requests) or scheduler.has_unfinished:
            now = time.perf_counter() - start
            while submitted < len(requests) and arrivals[submitted] <= now:
                prompt, limit = requests[submitted]
                index_of[scheduler.add_request(prompt, max_new_tokens=limit, sampling=SamplingConfig())] = submitted
                submitted += 1
            if not scheduler.has_unfinished:
                time.sleep(max(0.0, min(arrivals[submitted] - now, 0.001)))
                continue
            events = scheduler.step()
            steps += 1
            now = time.perf_counter() - start      # the step's tokens have been read back by now
            for index, event in events:
                request = index_of[index]
                if event.token_id is not None:
                    generated += 1
                    first.setdefault(request, now)
                if event.finish_reason is not None:
                    finish[request] = now
        engine.synchronize()
    assert len(finish) == len(requests), "every request must finish"
    return {
        "makespan": max(finish.values()), "generated": generated, "steps": steps,
        "ttft": [first[i] - arrivals[i] for i in range(len(requests))],
        "latency": [finish[i] - arrivals[i] for i in range(len(requests))],
    }


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    import numpy as np

    from .. import Engine
    from ..config import config_from_dict

    raw = dict(SHAPES[args.shape])
    full_layers = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    config = config_from_dict(raw)
    rng = np.random.default_rng(args.seed)
    requests = draw_requests(rng, config.vocab_size, args.requests, args.prompt_tokens, args.new_tokens)
    for prompt, limit in requests:
        if len(prompt) + limit > args.max_seq_len:
            print(f"error: a request of {len(prompt)} + {limit} tokens exceeds --max-seq-len {args.max_seq_len}", file=sys.stderr)
            return 2
    engine = Engine.from_config(config, seed=args.seed, dtype=args.dtype, max_seq_len=args.max_seq_len,
                                max_batch_size=args.max_batch_size, max_num_batched_tokens=args.step_tokens)
    interval = args.interval_ms / 1000.0
    for _ in range(args.warmups):
        run_once(engine, requests, interval)
        print("warm-up run done", file=sys.stderr, flush=True)
    runs = [run_once(engine, requests, interval) for _ in range(max(1, args.repeats))]

    def stat(key: str, fraction: float) -> float:
        return round(1000.0 * statistics.median(percentile(run[key], fraction) for run in runs), 1)

    makespan = statistics.median(run["makespan"] for run in runs)
    prompt_tokens = sum(len(p) for p, _ in requests)
    print(json.dumps({
        "workload": "staggered arrivals, continuous batching with chunked prefill",
        "shape": args.shape, "layers": config.num_hidden_layers, "layers_of_shape": full_layers, "dtype": args.dtype,
        "requests": args.requests, "interval_ms": args.interval_ms, "max_batch_size": args.max_batch_size,
        "step_tokens": args.step_tokens, "max_seq_len": args.max_seq_len,
        "prompt_tokens": prompt_tokens, "generated_tokens": runs[0]["generated"], "steps": runs[0]["steps"],
        "makespan_s": round(makespan, 3),
        "output_tok_s": round(statistics.median(run["generated"] / run["makespan"] for run in runs), 1),
        "total_tok_s": round(statistics.median((prompt_tokens + run["generated"]) / run["makespan"] for run in runs), 1),
        "ttft_ms_p50": stat("ttft", 0.5), "ttft_ms_p95": stat("ttft", 0.95),
        "latency_ms_p50": stat("latency", 0.5), "latency_ms_p95": stat("latency", 0.95),
        "data": "synthetic (seeded uniform random token ids and lengths, random weights)",
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
