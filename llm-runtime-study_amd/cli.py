"""Command line: `python -m llm_runtime_study_amd --model DIR --prompt TEXT`.

Options, defaults and output follow the reference's command line (mini_llm/cli.py:32-64
parser, 101-158 one prompt, 161-210 interactive, 213-247 metrics, 250-284 error handling:
typed errors print `error: ...` and exit with 2).  Added: --prompt-ids for models without
a tokenizer, --max-batch-size, --page-size, --no-graph, --decode-steps-per-launch.
"""

from __future__ import annotations

import argparse
import sys
import time
from dataclasses import dataclass
from pathlib import Path
from typing import Sequence, TextIO

from .errors import (CheckpointError, ConfigError, EngineError, GenerationError, KernelError, KVCacheError,
                     SamplingError, TokenizerError)
from .sampling import SamplingConfig
from .text import ChatMessage


@dataclass(frozen=True)
class RunMetrics:
    prompt_tokens: int
    generated_tokens: int
    time_to_first_token: float
    decode_seconds: float
    finish_reason: str


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="python -m llm_runtime_study_amd",
                                     description="Run a supported model with the MI355X inference runtime.")
    parser.add_argument("--model", type=Path, required=True)
    parser.add_argument("--prompt", help="raw prompt for one-shot mode, or an optional first interactive prompt")
    parser.add_argument("--prompt-ids", help="comma-separated token ids instead of a text prompt")
    parser.add_argument("--interactive", action="store_true", help="load the model once and repeatedly read prompts")
    parser.add_argument("--max-new-tokens", type=int, default=128)
    parser.add_argument("--max-seq-len", type=int, default=4096)
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-k", type=int)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--seed", type=int)
    parser.add_argument("--device", choices=("auto", "cpu", "mps", "cuda"), default="auto")
    parser.add_argument("--dtype", choices=("auto", "float16", "bfloat16", "float32"), default="auto")
    parser.add_argument("--thinking", action="store_true")
    parser.add_argument("--no-stream", action="store_true")
    parser.add_argument("--no-metrics", action="store_true")
    parser.add_argument("--max-batch-size", type=int, default=1)
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--no-graph", action="store_true", help="run decode steps without HIP graph replay")
    parser.add_argument("--decode-steps-per-launch", type=int, default=4,
                        help="greedy decode steps run from one graph launch; tokens then arrive that many at a time (1: one by one)")
    return parser


def _sampling_from_args(args) -> SamplingConfig:
    return SamplingConfig(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, seed=args.seed)


def _engine_from_args(args):
    from .engine.engine import Engine

    return Engine.from_model_dir(args.model, device=args.device, dtype=args.dtype, max_seq_len=args.max_seq_len,
                                 max_batch_size=args.max_batch_size, use_cuda_graph=not args.no_graph,
                                 page_size=args.page_size, decode_steps_per_launch=args.decode_steps_per_launch)


def _prompt_from_args(args, text: str | None):
    if args.prompt_ids is not None and text is None:
        try:
            return [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
        except ValueError as exc:
            raise GenerationError("--prompt-ids must be comma-separated integers") from exc
    return [ChatMessage(role="user", content=text)]


def run(args, *, output: TextIO) -> RunMetrics:
    if args.prompt is None and args.prompt_ids is None:
        raise GenerationError("--prompt is required unless --interactive is used")
    sampling = _sampling_from_args(args)
    engine = _engine_from_args(args)
    return _run_prompt(engine, _prompt_from_args(args, args.prompt), args, sampling=sampling, output=output)


def _run_prompt(engine, prompt, args, *, sampling, output: TextIO, include_load_time: bool = True) -> RunMetrics:
    started = time.perf_counter()
    stream = engine.generate((prompt,), max_new_tokens=args.max_new_tokens, sampling=sampling, enable_thinking=args.thinking)
    events, first_token = [], None
    for _, event in stream:
        if first_token is None:
            first_token = time.perf_counter()
        events.append(event)
        if not args.no_stream:
            if event.text_delta:
                print(event.text_delta, end="", flush=True, file=output)
            elif engine.tokenizer is None and event.token_id is not None:
                print(event.token_id, end=" ", flush=True, file=output)
    finished = time.perf_counter()
    if not events:
        raise GenerationError("generation ended without a terminal event")
    prompt_tokens = events[0].prompt_token_count
    if prompt_tokens is None:
        raise GenerationError("first generation event is missing prompt-token count")
    if args.no_stream:
        text = events[-1].text if engine.tokenizer is not None else " ".join(str(e.token_id) for e in events if e.token_id is not None)
        print(text, file=output)
    else:
        print(file=output)
    metrics = RunMetrics(
        prompt_tokens=prompt_tokens,
        generated_tokens=sum(e.token_id is not None for e in events),
        time_to_first_token=(first_token or finished) - started,
        decode_seconds=sum(e.model_seconds or 0.0 for e in events[1:]),
        finish_reason=events[-1].finish_reason or "unknown",
    )
    if not args.no_metrics:
        _print_metrics(engine, metrics, output=output, include_load_time=include_load_time)
    return metrics


def run_interactive(args, *, input_stream: TextIO, output: TextIO, error: TextIO) -> None:
    sampling = _sampling_from_args(args)
    engine = _engine_from_args(args)
    print(f"Loaded model on {engine.device} with {engine.dtype} in {engine.load_seconds:.2f} s.", file=output)
    print("Enter a prompt. Use /quit or /exit to stop.", file=output)
    first = args.prompt
    while True:
        if first is not None:
            prompt, first = first, None
            print(f"you> {prompt}", file=output)
        else:
            print("you> ", end="", flush=True, file=output)
            prompt = input_stream.readline()
            if prompt == "":
                print(file=output)
                return
            prompt = prompt.rstrip("\r\n")
        if prompt.strip() in {"/quit", "/exit"}:
            return
        if not prompt.strip():
            continue
        print("assistant> ", end="", flush=True, file=output)
        try:
            _run_prompt(engine, [ChatMessage(role="user", content=prompt)], args, sampling=sampling, output=output,
                        include_load_time=False)
        except (GenerationError, KVCacheError) as exc:
            print(file=output)
            print(f"error: {exc}", file=error)


def _print_metrics(engine, metrics: RunMetrics, *, output: TextIO, include_load_time: bool = True) -> None:
    cache_text = "not allocated"
    if engine.last_cache_capacity:
        cache_text = f"{engine.last_cache_num_bytes / (1024 ** 2):.2f} MiB ({engine.last_cache_capacity} positions)"
    decode_tokens = max(0, metrics.generated_tokens - 1)
    rate = decode_tokens / metrics.decode_seconds if decode_tokens and metrics.decode_seconds > 0 else None
    print("\nmetrics", file=output)
    print(f"  device:              {engine.device}", file=output)
    print(f"  dtype:               {engine.dtype}", file=output)
    if include_load_time:
        print(f"  load time:           {engine.load_seconds:.2f} s", file=output)
    print(f"  prompt tokens:       {metrics.prompt_tokens}", file=output)
    print(f"  generated tokens:    {metrics.generated_tokens}", file=output)
    print(f"  cache:               {cache_text}", file=output)
    print(f"  time to first token: {metrics.time_to_first_token * 1_000:.2f} ms", file=output)
    print(f"  decode throughput:   {'n/a' if rate is None else f'{rate:.2f} tokens/s'}", file=output)
    print(f"  stop reason:         {metrics.finish_reason}", file=output)


def main(argv: Sequence[str] | None = None, *, input_stream: TextIO | None = None, output: TextIO | None = None,
         error: TextIO | None = None) -> int:
    input_stream = sys.stdin if input_stream is None else input_stream
    output = sys.stdout if output is None else output
    error = sys.stderr if error is None else error
    args = build_parser().parse_args(argv)
    try:
        if args.interactive:
            run_interactive(args, input_stream=input_stream, output=output, error=error)
        else:
            run(args, output=output)
    except KeyboardInterrupt:
        print("\nInterrupted.", file=output)
    except (CheckpointError, ConfigError, EngineError, GenerationError, KVCacheError, KernelError, SamplingError,
            TokenizerError) as exc:
        print(f"error: {exc}", file=error)
        return 2
    return 0
