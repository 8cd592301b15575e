"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and owns no forward pass, cache or loader: it drives the same model,
step function, cache manager and kernels that generation uses.

Input, one JSON object a line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step form one batch.  A request is admitted when its id is first seen and
gives everything back when it is listed in `end`.  For a step in which logits are wanted,
`<out>/<step>.f32` holds them as little-endian float32 [wanted, vocab], in the order of the
entries and of `want`.  After every step a line `done <step>` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

import torch

from ..cache import CacheManager
from ..errors import GenerationError
from .loading import load_model, resolve_device, resolve_dtype
from .step import ModelRunner, StepEntry

PAGE_SIZE = 16
MAX_LIVE_REQUESTS = 8


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="trace_run", description="Replay token ids through the model and dump logits.")
    parser.add_argument("--model", type=Path, required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), required=True)
    parser.add_argument("--out", type=Path, required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens that live requests hold at any time; the cache pool is made for this many")
    parser.add_argument("--page-size", type=int, default=PAGE_SIZE)
    return parser


def make_runner(model_dir, dtype_name: str, max_tokens: int, page_size: int = PAGE_SIZE, library_gemm: bool = True,
                use_graph: bool = False):
    device = resolve_device("auto")
    dtype = resolve_dtype(dtype_name)
    # a replay takes the folder as it is: tensors stored in 32-bit beside bfloat16 ones stay 32-bit
    config, model = load_model(model_dir, dtype, device, stored_precision=True)
    if max_tokens <= 0:
        raise GenerationError("--max-tokens must be positive")
    num_pages = -(-max_tokens // page_size)
    cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=num_pages, max_requests=MAX_LIVE_REQUESTS,
                         max_seq_len=min(model.spec.max_positions, num_pages * page_size), dtype=dtype, device=device)
    runner = ModelRunner(model, cache, max_step_tokens=num_pages * page_size, dtype=dtype, device=device, library_gemm=library_gemm,
                         use_graph=use_graph)
    return runner


def replay(runner: ModelRunner, lines, out_dir: Path, echo=print) -> None:
    out_dir.mkdir(parents=True, exist_ok=True)
    live: dict = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            key = item["id"]
            if key not in live:
                live[key] = runner.cache.admit(key)
            entries.append(StepEntry(live[key], [int(t) for t in item["tokens"]], [int(w) for w in item.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                logits.cpu().numpy().astype("<f4").tofile(out_dir / f"{step}.f32")
        for key in record.get("end", []):
            if key in live:
                runner.cache.release(live.pop(key))
        echo(f"done {step}")


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    runner = make_runner(args.model, args.dtype, args.max_tokens, args.page_size)
    with torch.cuda.device(runner.device):
        replay(runner, sys.stdin, args.out, echo=lambda text: print(text, flush=True))
        torch.cuda.synchronize()
    return 0
