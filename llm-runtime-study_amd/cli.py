"""Command line: `python -m llm_runtime_study_amd --model DIR --prompt TEXT`.

What a user of the reference's command line finds again (mini_llm/cli.py:32-64 options and
defaults, 213-247 the metrics block, 250-284 typed errors print `error: ...` and exit with 2):
the option names and defaults, the streamed answer followed by the metrics block, the
interactive loop with /quit and /exit.  Added here: --prompt-ids for model folders without a
tokenizer, --random-weights SEED for a folder that holds only a config.json, --device hip,
--max-batch-size, --page-size, --no-graph, --decode-steps-per-launch.

A run is one Session: it owns the engine and the sampling settings, answers prompts one at a
time and keeps a Tally of each answer (token counts and the times the metrics block reports).
One-shot and interactive mode differ only in where the prompts come from.
"""

from __future__ import annotations

import argparse
import sys
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Iterable, Sequence, TextIO

from .errors import (CheckpointError, ConfigError, EngineError, GenerationError, KernelError, KVCacheError,
                     SamplingError, TokenizerError)
from .sampling import SamplingConfig
from .text import ChatMessage

REPORTED_ERRORS = (CheckpointError, ConfigError, EngineError, GenerationError, KVCacheError, KernelError, SamplingError,
                   TokenizerError)
LEAVE_WORDS = ("/quit", "/exit")

# flag, then what argparse is told about it; the first block is the reference's, the second this runtime's own
OPTIONS = (
    ("--model", dict(type=Path, required=True)),
    ("--prompt", dict(help="raw prompt for one-shot mode, or an optional first interactive prompt")),
    ("--interactive", dict(action="store_true", help="load the model once and repeatedly read prompts")),
    ("--max-new-tokens", dict(type=int, default=128)),
    ("--max-seq-len", dict(type=int, default=4096)),
    ("--temperature", dict(type=float, default=0.0)),
    ("--top-k", dict(type=int)),
    ("--top-p", dict(type=float, default=1.0)),
    ("--seed", dict(type=int)),
    ("--device", dict(choices=("auto", "cpu", "mps", "cuda", "hip"), default="auto")),
    ("--dtype", dict(choices=("auto", "float16", "bfloat16", "float32"), default="auto")),
    ("--thinking", dict(action="store_true")),
    ("--no-stream", dict(action="store_true")),
    ("--no-metrics", dict(action="store_true")),

    ("--prompt-ids", dict(help="comma-separated token ids instead of a text prompt")),
    ("--random-weights", dict(type=int, metavar="SEED",
                              help="draw the weights from this seed; --model then needs to hold a config.json only")),
    ("--max-batch-size", dict(type=int, default=1)),
    ("--page-size", dict(type=int, default=16)),
    ("--no-graph", dict(action="store_true", help="run decode steps without HIP graph replay")),
    ("--decode-steps-per-launch", dict(type=int, default=4, help="greedy decode steps run from one graph launch; tokens "
                                                                "then arrive that many at a time (1: one by one)")),
)


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="python -m llm_runtime_study_amd",
                                     description="Run a supported model with the MI355X inference runtime.")
    for flag, settings in OPTIONS:
        parser.add_argument(flag, **settings)
    return parser


def open_engine(args):
    """The engine the options ask for: the folder's checkpoint, or random weights for its config.json."""
    from .engine.engine import Engine

    shared = dict(device=args.device, dtype=args.dtype, max_seq_len=args.max_seq_len, max_batch_size=args.max_batch_size,
                  use_cuda_graph=not args.no_graph, page_size=args.page_size, decode_steps_per_launch=args.decode_steps_per_launch)
    if args.random_weights is None:
        return Engine.from_model_dir(args.model, **shared)
    if args.random_weights < 0:
        raise EngineError("--random-weights needs a non-negative seed")
    from .config import chat_template_for, load_config
    from .text import TextTokenizer

    config = load_config(args.model)
    tokenizer = TextTokenizer.from_model_dir(args.model, config.vocab_size, chat_template_for(config))
    return Engine.from_config(config, seed=args.random_weights, tokenizer=tokenizer, **shared)


def token_ids_from(text: str) -> list[int]:
    try:
        return [int(piece) for piece in text.replace(",", " ").split()]
    except ValueError as exc:
        raise GenerationError("--prompt-ids must be comma-separated integers") from exc


@dataclass
class Tally:
    """What one answer amounted to; filled while its events stream by."""

    asked_at: float
    prompt_tokens: int | None = None
    generated_tokens: int = 0
    first_event_at: float | None = None
    done_at: float | None = None
    decode_seconds: float = 0.0          # model time of every event after the first
    finish_reason: str = "unknown"
    text: str = ""
    token_ids: list = field(default_factory=list)
    events: int = 0

    def take(self, event) -> None:
        now = time.perf_counter()
        if self.events == 0:
            self.first_event_at = now
            self.prompt_tokens = event.prompt_token_count
        else:
            self.decode_seconds += event.model_seconds or 0.0
        self.events += 1
        if event.token_id is not None:
            self.generated_tokens += 1
            self.token_ids.append(event.token_id)
        self.text = event.text
        if event.finish_reason is not None:
            self.finish_reason = event.finish_reason
        self.done_at = now

    def close(self) -> None:
        if self.events == 0:
            raise GenerationError("generation ended without a terminal event")
        if self.prompt_tokens is None:
            raise GenerationError("first generation event is missing prompt-token count")

    @property
    def time_to_first_token(self) -> float:
        return (self.first_event_at or self.done_at or self.asked_at) - self.asked_at

    @property
    def decode_rate(self) -> float | None:
        steps = self.generated_tokens - 1
        return steps / self.decode_seconds if steps > 0 and self.decode_seconds > 0 else None


class Session:
    def __init__(self, args, engine, sampling: SamplingConfig, *, output: TextIO, error: TextIO):
        self.args, self.engine, self.sampling, self.output, self.error = args, engine, sampling, output, error

    @classmethod
    def open(cls, args, *, output: TextIO, error: TextIO) -> "Session":
        """Checks what can be checked before the model is loaded (the prompt's presence, the sampling
        settings), then loads it."""
        if not args.interactive and args.prompt is None and args.prompt_ids is None:
            raise GenerationError("--prompt is required unless --interactive is used")
        sampling = SamplingConfig(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, seed=args.seed)
        return cls(args, open_engine(args), sampling, output=output, error=error)

    def say(self, text: str = "", end: str = "\n") -> None:
        print(text, end=end, flush=True, file=self.output)

    # ------------------------------------------------------------- one answer
    def answer(self, prompt, *, with_load_time: bool) -> Tally:
        """Generate for one prompt (chat messages or token ids), showing tokens as they come unless
        --no-stream, then the metrics block unless --no-metrics."""
        args, has_text = self.args, self.engine.tokenizer is not None
        tally = Tally(asked_at=time.perf_counter())
        events = self.engine.generate((prompt,), max_new_tokens=args.max_new_tokens, sampling=self.sampling,
                                      enable_thinking=args.thinking)
        for _, event in events:
            tally.take(event)
            if args.no_stream:
                continue
            if has_text:
                self.say(event.text_delta, end="")
            elif event.token_id is not None:
                self.say(str(event.token_id), end=" ")
        tally.close()
        if args.no_stream:
            self.say(tally.text if has_text else " ".join(map(str, tally.token_ids)))
        else:
            self.say()
        if not args.no_metrics:
            for line in self.metrics_lines(tally, with_load_time):
                self.say(line)
        return tally

    def metrics_lines(self, tally: Tally, with_load_time: bool) -> Iterable[str]:
        engine = self.engine
        cache = "not allocated"
        if engine.last_cache_capacity:
            cache = f"{engine.last_cache_num_bytes / 2 ** 20:.2f} MiB ({engine.last_cache_capacity} positions)"
        rate = tally.decode_rate
        rows = [("device", f"{engine.device}"), ("dtype", f"{engine.dtype}")]
        if with_load_time:
            rows.append(("load time", f"{engine.load_seconds:.2f} s"))
        rows += [("prompt tokens", f"{tally.prompt_tokens}"), ("generated tokens", f"{tally.generated_tokens}"), ("cache", cache),
                 ("time to first token", f"{tally.time_to_first_token * 1e3:.2f} ms"),
                 ("decode throughput", "n/a" if rate is None else f"{rate:.2f} tokens/s"), ("stop reason", tally.finish_reason)]
        yield "\nmetrics"
        for name, value in rows:
            yield f"  {name + ':':<21}{value}"

    # --------------------------------------------------------------- the modes
    def one_shot(self) -> Tally:
        args = self.args
        if args.prompt is not None:
            prompt = [ChatMessage("user", args.prompt)]
        else:
            prompt = token_ids_from(args.prompt_ids)
        return self.answer(prompt, with_load_time=True)

    def prompts_from(self, lines: TextIO) -> Iterable[str]:
        """The first prompt from --prompt if given, then one per line read; ends at end of input or a leave word."""
        if self.args.prompt is not None:
            self.say(f"you> {self.args.prompt}")
            yield self.args.prompt
        while True:
            self.say("you> ", end="")
            line = lines.readline()
            if not line:
                self.say()
                return
            yield line.rstrip("\r\n")

    def converse(self, lines: TextIO) -> None:
        engine = self.engine
        self.say(f"Loaded model on {engine.device} with {engine.dtype} in {engine.load_seconds:.2f} s.")
        self.say("Enter a prompt. Use /quit or /exit to stop.")
        for prompt in self.prompts_from(lines):
            wanted = prompt.strip()
            if wanted in LEAVE_WORDS:
                return
            if not wanted:
                continue
            self.say("assistant> ", end="")
            try:
                self.answer([ChatMessage("user", prompt)], with_load_time=False)
            except (GenerationError, KVCacheError) as exc:      # this prompt failed; the session goes on
                self.say()
                print(f"error: {exc}", file=self.error)


def main(argv: Sequence[str] | None = None, *, input_stream: TextIO | None = None, output: TextIO | None = None,
         error: TextIO | None = None) -> int:
    output = output or sys.stdout
    error = error or sys.stderr
    args = build_parser().parse_args(argv)
    try:
        session = Session.open(args, output=output, error=error)
        if args.interactive:
            session.converse(input_stream or sys.stdin)
        else:
            session.one_shot()
    except KeyboardInterrupt:
        print("\nInterrupted.", file=output)
    except REPORTED_ERRORS as exc:
        print(f"error: {exc}", file=error)
        return 2
    return 0
