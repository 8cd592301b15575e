"""Host time of a mixed step: how long the process needs to enqueue one step of a prompt portion beside
single tokens of decoding requests, against how long the GPU needs to run it.

    python -m llm_runtime_study_amd.benchmarks.host_cost [--shape 8b] [--tokens 512] [--decoding 8]
        [--context 300] [--layers L] [--repeats 6] [--seed 0]

Three ways of launching the same step are timed in turn, each with a runner of its own over the same
weights: through the parts (every launch made by Python), from a recorded launch plan (one call into the
library makes them all again), and from the HIP graph that a plan is captured into once it has come back
a few times.  Host time is the wall clock from the call of the step function to its return; total time
adds the wait for the GPU.  One JSON line.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time

from .shapes import SHAPES


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="host_cost", description=__doc__.splitlines()[0])
    parser.add_argument("--shape", choices=tuple(SHAPES), default="8b")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (reported)")
    parser.add_argument("--tokens", type=int, default=512, help="length of the prompt portion")
    parser.add_argument("--decoding", type=int, default=8, help="requests bringing one token each beside it")
    parser.add_argument("--context", type=int, default=300, help="tokens each decoding request already holds")
    parser.add_argument("--repeats", type=int, default=6)
    parser.add_argument("--seed", type=int, default=0)
    return parser


def measure(engine, runner, args, rng, repeats: int, warmups: int) -> dict:
    """Median host and total milliseconds of `repeats` steps of the same shape, after `warmups` untimed ones."""
    import torch

    from ..engine.step import StepEntry

    vocab = engine.config.vocab_size
    with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
        others = [runner.cache.admit(f"decoding-{i}") for i in range(args.decoding)]
        for cache in others:                     # their contexts, one request a step (a step's token budget)
            runner.step([StepEntry(cache, rng.integers(0, vocab, args.context).tolist(), [])])
        host, total = [], []
        for i in range(warmups + repeats):
            cache = runner.cache.admit(f"prompt-{i}")
            entries = [StepEntry(c, [5], [0]) for c in others]
            entries.append(StepEntry(cache, rng.integers(0, vocab, args.tokens).tolist(), [args.tokens - 1]))
            engine.synchronize()
            begun = time.perf_counter()
            runner.step(entries)
            returned = time.perf_counter()
            engine.synchronize()
            finished = time.perf_counter()
            runner.cache.release(cache)
            for c in others:                     # the same shape again next time
                runner.cache.rollback(c, c.length - 1)
            if i >= warmups:
                host.append((returned - begun) * 1e3)
                total.append((finished - begun) * 1e3)
        for cache in others:
            runner.cache.release(cache)
    return {"host_ms": round(statistics.median(host), 3), "total_ms": round(statistics.median(total), 3)}


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("host_cost: needs the GPU", file=sys.stderr)
        return 2
    from .. import Engine
    from ..config import config_from_dict
    from ..engine.step import ModelRunner

    shape = dict(SHAPES[args.shape])
    layers_of_shape = shape["num_hidden_layers"]
    if args.layers is not None:
        shape["num_hidden_layers"] = args.layers
    config = config_from_dict(shape)
    engine = Engine.from_config(config, seed=args.seed, dtype="bfloat16", max_seq_len=4096, max_batch_size=args.decoding + 2,
                                max_num_batched_tokens=max(2048, args.tokens + args.decoding))
    result = {"workload": "host time of one mixed step", "shape": args.shape, "layers": config.num_hidden_layers,
              "layers_of_shape": layers_of_shape, "prompt_tokens": args.tokens, "decoding_requests": args.decoding,
              "context_of_each": args.context, "repeats": args.repeats}
    rng = np.random.default_rng(args.seed)
    stock = engine.runner

    def runner_like_the_engines(use_plans: bool) -> ModelRunner:
        with torch.cuda.device(engine.device), torch.cuda.stream(engine.stream):
            return ModelRunner(stock.model, stock.cache, max_step_tokens=stock.max_step_tokens, dtype=stock.dtype,
                               device=stock.device, use_graph=False, kernels=stock.kernels, use_plans=use_plans)

    # through the parts: plans switched off
    parts = runner_like_the_engines(False)
    result["through_parts"] = measure(engine, parts, args, rng, args.repeats, 2)
    # from the plan: it is recorded in the warm-up and never used often enough to be captured
    planned = runner_like_the_engines(True)
    planned.PLAN_GRAPH_AFTER = 1 << 30
    result["from_plan"] = dict(measure(engine, planned, args, rng, args.repeats, 2), recordings=planned.plan_recordings, replays=planned.plan_replays)
    # from the graph of the plan
    graphed = runner_like_the_engines(True)
    result["from_graph_of_plan"] = dict(measure(engine, graphed, args, rng, args.repeats, 2 + graphed.PLAN_GRAPH_AFTER),
                                        recordings=graphed.plan_recordings, replays=graphed.plan_replays,
                                        graph_replays=graphed.plan_graph_replays)
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
