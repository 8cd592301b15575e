"""Decode and prefill throughput of the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048] [--layers L] [--shape 8b|14b|32b]

A step is one decode step of the whole engine (scheduler, step function, sampling) at the
given batch; `value` is decoded tokens per second.  The same line carries the prefill rate
of one 2,048-token prompt, the decode step's achieved HBM bandwidth (bytes it must read:
every weight once plus the cache of the live requests) and decode rates at batch 1 and 64.
Peaks are MI355X's published ones: HBM 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

from llm_runtime_study_amd.benchmarks.shapes import QWEN3_8B, SHAPES  # noqa: E402  (layer sizes of the 8B, 14B and 32B models)

FULL_LAYERS = QWEN3_8B["num_hidden_layers"]
BENCHMARK_CONTEXT = 4096      # tokens a request's cache can hold at the least: the benchmark context of the 8B configuration
PORTION_TOKENS = 512          # a second prefill figure: the size of a prompt portion in the serving configuration
SIZE_KEYS = ("hidden_size", "intermediate_size", "num_attention_heads", "num_key_value_heads", "head_dim", "vocab_size")


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=2048)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--max-seq-len", type=int, default=None, help="context the cache is made for: 4,096 (the benchmark context of the 8B configuration) or what the workload needs, whichever is more")
    parser.add_argument("--num-pages", type=int, default=None, help="pages of the cache pool (default: max-seq-len tokens for every request of the largest batch)")
    parser.add_argument("--shape", choices=tuple(SHAPES), default="8b", help="layer sizes: Qwen3-8B (default), 14B or 32B")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (reported in config)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--temperature", type=float, default=0.0, help="draw the tokens at this temperature instead of taking the largest logit (reported in config)")
    parser.add_argument("--top-k", type=int, default=None, help="with --temperature: keep the k likeliest tokens")
    parser.add_argument("--top-p", type=float, default=1.0, help="with --temperature: keep the likeliest tokens up to this share of the mass")
    parser.add_argument("--no-graph", action="store_true")
    parser.add_argument("--decode-steps-per-launch", type=int, default=4, help="greedy decode steps run from one graph launch (1: one step a launch)")
    parser.add_argument("--plain-deal", action="store_true", help="the product for 17..64 rows never deals its weight rows evenly (every workgroup 16 rows a wave)")
    parser.add_argument("--no-reserve", action="store_true", help="let every tensor be an allocation of its own instead of one segment for the engine")
    parser.add_argument("--no-launch-ahead", action="store_true", help="wait for a launch's tokens before the next launch is queued")
    parser.add_argument("--library-mid-gemm", action="store_true", help="products of 17..128 rows through the vendor library instead of this package's kernel for them")
    parser.add_argument("--own-gemm", action="store_true", help="this package's kernel also for products of many rows (default: vendor library)")
    return parser.parse_args()


def prefill_flops(model, tokens: int) -> float:
    """Matrix products of every layer for all tokens of a prompt read from its start (each part says its own: projections,
    causal attention), and the head for one row."""
    return model.flops(tokens, tokens * (tokens + 1) // 2, 1)


def decode_lead(batch: int, context: int, step_tokens: int) -> int:
    """Tokens the first request has decoded when the last one has read its prompt: prompts are read one
    after the other, in portions of at most `step_tokens`, and whoever has finished decodes meanwhile."""
    return (batch - 1) * -(-context // step_tokens)


def warmup_room(warmup: int, per_launch: int) -> int:
    """Most decode steps the warm-up of measure_decode() takes (its rounds go on until no new graph is captured)."""
    return 6 * (-(-max(warmup, 1) // per_launch) * per_launch + 2 * per_launch) + per_launch


def measure_decode(engine, batch: int, context: int, steps: int, warmup: int, seed: int, sampling=None):
    """Prefill `batch` prompts of `context` random tokens through the scheduler, then time `steps`
    decode steps.  Returns (seconds per step list, mean context length over the timed steps)."""
    import numpy as np
    import torch

    from llm_runtime_study_amd import SamplingConfig

    rng = np.random.default_rng(seed)
    vocab = engine.config.vocab_size
    scheduler = engine.create_scheduler(ignore_eos=True)   # every request runs to its length limit
    # a request decodes while the prompts behind it are still read, one portion a step
    lead = decode_lead(batch, context, engine.max_num_batched_tokens)
    for _ in range(batch):
        scheduler.add_request(rng.integers(0, vocab, context).tolist(),
                              max_new_tokens=steps + lead + batch + 8 + warmup_room(warmup, scheduler.decode_steps_per_launch),
                              sampling=sampling if sampling is not None else SamplingConfig())
    times = []
    with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
        # prefill phase: until every request has sampled its first token
        produced = 0
        while produced < batch:
            produced += sum(1 for _, e in scheduler.step() if e.prompt_token_count is not None)
        # one call of the scheduler may hold several decode steps (one graph launch): count steps, not calls.  With
        # launches queued ahead a call returns the tokens of the launch queued by the call before it, and queues the next:
        # the settings below are changed so that exactly `count` steps run, none queued when the last call returns.
        per_launch, ahead = scheduler.decode_steps_per_launch, scheduler.launch_ahead
        runner = engine.runner

        def run(count: int, record: bool) -> None:
            done = 0
            while done < count:
                if scheduler.steps_in_flight == 0:     # this call queues a launch and, ahead, one of the same size behind it
                    scheduler.launch_ahead = ahead and count - done >= 2 * per_launch
                    scheduler.decode_steps_per_launch = min(per_launch, count - done)
                else:                                  # this call queues what may still be queued behind the launch in flight
                    left = count - done - scheduler.steps_in_flight
                    scheduler.launch_ahead = ahead and left > 0
                    scheduler.decode_steps_per_launch = max(1, min(per_launch, left))
                started = time.perf_counter()
                events = scheduler.step()
                elapsed = time.perf_counter() - started                # the call returns when its launch's tokens are there
                assert len(events) % batch == 0 and len(events) > 0
                held = len(events) // batch
                if record:
                    times.extend([elapsed / held] * held)
                done += held
            assert done == count and scheduler.steps_in_flight == 0
            scheduler.launch_ahead, scheduler.decode_steps_per_launch = ahead, per_launch

        # warm-up: at least `warmup` steps, in whole launches, until a round of launches captures no new graph (a launch
        # that follows another, and each of the two result buffers, has a graph of its own), and one launch of every
        # size the timed steps will use
        warmed = 0
        for _ in range(6):
            captured = runner.graph_captures
            rounds = -(-max(warmup, 1) // per_launch) * per_launch + (2 * per_launch if ahead else 0)
            run(rounds, False)
            warmed += rounds
            if runner.graph_captures == captured:
                break
        if steps % per_launch:
            run(steps % per_launch, False)
            warmed += steps % per_launch
        engine.synchronize()
        run(steps, True)
        engine.synchronize()
        assert len(times) == steps
        scheduler.abort_all()
    # requests finished their prompts `portions` steps apart, so they are up to `lead` tokens apart in length
    mean_context = context + 1 + warmed + lead / 2 + (steps - 1) / 2
    return times, mean_context


def measure_prefill(engine, tokens: int, repeats: int, seed: int):
    """Seconds from handing the scheduler one prompt of `tokens` tokens to its first token, `repeats` times
    (after one untimed run): admission, the step function on the whole prompt, the token's choice."""
    import numpy as np
    import torch

    rng = np.random.default_rng(seed)
    times = []
    scheduler = engine.create_scheduler(ignore_eos=True)
    with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
        for _ in range(repeats + 1):
            scheduler.add_request(rng.integers(0, engine.config.vocab_size, tokens).tolist(), max_new_tokens=1)
            engine.synchronize()
            started = time.perf_counter()
            events = []
            while scheduler.has_unfinished:
                events += scheduler.step()
            engine.synchronize()
            times.append(time.perf_counter() - started)
            assert len(events) == 1 and events[0][1].prompt_token_count == tokens
    return times[1:]  # the first run warms up buffers


def prefill_entry(engine, tokens: int, dtype_name: str, seed: int) -> dict:
    seconds = statistics.median(measure_prefill(engine, tokens, repeats=3, seed=seed))
    return {"value": round(tokens / seconds, 1), "tokens": tokens, "ms": round(seconds * 1e3, 3),
            "frac": round(prefill_flops(engine.model, tokens) / seconds / FLOP_PEAK[dtype_name], 4)}


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    import torch

    from llm_runtime_study_amd import Engine
    from llm_runtime_study_amd.config import config_from_dict

    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    raw = dict(SHAPES[args.shape], num_hidden_layers=args.layers)
    config = config_from_dict(raw)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    needed = (args.context + args.steps + warmup_room(args.warmup, max(args.decode_steps_per_launch, 1))
              + decode_lead(max_batch, args.context, max(2048, args.prefill_tokens)) + max_batch + 64)
    needed = max(needed, args.prefill_tokens + 1)
    max_seq_len = max(needed, BENCHMARK_CONTEXT) if args.max_seq_len is None else args.max_seq_len
    if max_seq_len < needed:
        print(f"bench.py: --max-seq-len {max_seq_len} is less than the {needed} tokens the workload needs", file=sys.stderr)
        return 2
    from llm_runtime_study_amd.kernels.ops import KernelChoice

    engine = Engine.from_config(config, seed=0, dtype=args.dtype, max_seq_len=max_seq_len, max_batch_size=max_batch,
                                max_num_batched_tokens=max(2048, args.prefill_tokens), use_cuda_graph=not args.no_graph, num_pages=args.num_pages,
                                kernels=KernelChoice(library=not args.own_gemm, mid=not args.library_mid_gemm, mid_even=1 if args.plain_deal else 0),
                                decode_steps_per_launch=args.decode_steps_per_launch, launch_ahead=not args.no_launch_ahead,
                                reserve_memory=not args.no_reserve)
    dtype_name = "bf16" if args.dtype == "bfloat16" else "fp32"

    prefill = prefill_entry(engine, args.prefill_tokens, dtype_name, seed=1)
    prefill_portion = prefill_entry(engine, PORTION_TOKENS, dtype_name, seed=5) if args.prefill_tokens != PORTION_TOKENS else prefill

    sampling = None
    if args.temperature > 0:
        from llm_runtime_study_amd import SamplingConfig

        sampling = SamplingConfig(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, seed=7)
    times, mean_context = measure_decode(engine, args.batch, args.context, args.steps, args.warmup, seed=2, sampling=sampling)
    total = sum(times)
    step_s = total / len(times)
    weight_bytes = engine.model.weight_bytes()
    kv_bytes = args.batch * mean_context * engine.cache_manager.bytes_per_token()
    achieved = (weight_bytes + kv_bytes) / step_s

    points = {}
    if not args.no_points:
        for batch in (1, 64):
            point_steps = min(args.steps, 64)
            t, _ = measure_decode(engine, batch, args.context, point_steps, min(args.warmup, 4), seed=3 + batch, sampling=sampling)
            points[f"decode_b{batch}"] = round(batch * len(t) / sum(t), 2)

    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-{args.shape.upper()} shape)",
        "value": round(args.batch * len(times) / total, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic (seeded uniform random token ids, random weights N(0, 0.02))",
        "config": {
            "model": f"Qwen3-{args.shape.upper()} shape", "layers": args.layers, "layers_of_shape": full_layers,
            **{key: raw[key] for key in SIZE_KEYS if key in raw},
            "global_batch": args.batch, "seq_len": args.context, "new_tokens": args.steps + args.warmup,
            "max_seq_len": max_seq_len, "num_pages": engine.cache_manager.groups[0].pool.num_pages, "page_size": engine.page_size,
            "prefill_tokens": args.prefill_tokens,
            "decode_steps_per_graph_launch": args.decode_steps_per_launch if engine.runner.use_graph else 0,
            "prefill_gemm": "own" if args.own_gemm else "hipBLASLt", "parallelism": "single GPU",
            "sampling": "greedy" if sampling is None else f"temperature {args.temperature} top_k {args.top_k} top_p {args.top_p}",
        },
        "prefill": prefill,
        f"prefill_{PORTION_TOKENS}": prefill_portion,
        "roofline": {
            "bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK, 4),
        },
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
