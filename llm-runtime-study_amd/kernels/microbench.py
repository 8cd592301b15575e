"""Timings of single kernels at the shapes of a model, outside any model.

    python -m llm_runtime_study_amd.kernels.microbench attention_prefill --tokens 2048,8192 --group 16,32
    python -m llm_runtime_study_amd.kernels.microbench attention_prefill --tokens 64 --before 32704 --key-splits 1,8,32
    python -m llm_runtime_study_amd.kernels.microbench attention_decode --batch 1,8,64 --context 2048 --splits 1,4,8
    python -m llm_runtime_study_amd.kernels.microbench gemm --rows 1,8,16,64,2048
    python -m llm_runtime_study_amd.kernels.microbench memory
    python -m llm_runtime_study_amd.kernels.microbench sampling --batch 8,64   # top-k / top-p filtering and the draw, a vocabulary of 151,936
    python -m llm_runtime_study_amd.kernels.microbench lds          # LDS read rate by the distance between a fragment's rows
    python -m llm_runtime_study_amd.kernels.microbench mfma         # matrix instructions with vector work beside them

Head and matrix shapes default to those of Qwen3-8B and can be changed with options.  Weights and
caches larger than the last-level cache are rotated between calls where a kernel streams them once
(decode attention, products of few rows), so that a timing is one of reads from memory.  Prints one
line per case; the profiler attaches to this program like to any other.
"""

from __future__ import annotations

import argparse
import math
import sys

import torch

from . import ops


def _ints(text: str) -> list[int]:
    return [int(part) for part in text.split(",") if part]


def _time(call, repeats: int) -> float:
    """Seconds per call of `call(i)`, measured over `repeats` calls after three warm-up calls."""
    for i in range(3):
        call(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(repeats):
        call(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / repeats * 1e-3


def attention_prefill(args) -> None:
    """One request's prompt, or a later portion of it: `tokens` queries after `before` cached tokens."""
    nq, nkv, d, page, before = args.heads, args.kv_heads, args.head_dim, args.page_size, args.before
    for tokens in _ints(args.tokens):
        pages = -(-(before + tokens) // page)
        k_pages = torch.randn(pages + 1, nkv, page, d, device="cuda", dtype=torch.bfloat16)
        v_pages = torch.randn(pages + 1, nkv, d, page, device="cuda", dtype=torch.bfloat16)
        table = torch.randperm(pages, device="cuda").to(torch.int32).view(1, -1)
        q = torch.randn(tokens, (nq + 2 * nkv) * d, device="cuda", dtype=torch.bfloat16)
        out = torch.empty(tokens, nq * d, device="cuda", dtype=torch.bfloat16)
        request = torch.zeros(tokens, dtype=torch.int32, device="cuda")
        positions = torch.arange(before, before + tokens, dtype=torch.int32, device="cuda")
        flops = 4 * (tokens * before + tokens * (tokens + 1) / 2) * nq * d
        groups = _ints(args.group) if args.group else [ops.attention_prefill_group(tokens)]
        for size in groups:
            starts = list(range(0, tokens, size))[::-1]          # longest contexts first, as the engine orders them
            token0 = torch.tensor(starts, dtype=torch.int32, device="cuda")
            count = torch.tensor([min(size, tokens - s) for s in starts], dtype=torch.int32, device="cuda")
            for splits in _ints(args.key_splits):
                part_o = torch.empty(tokens, nq * splits * d, device="cuda") if splits > 1 else None
                part_ml = torch.empty(tokens, nq * splits * 2, device="cuda") if splits > 1 else None
                seconds = _time(lambda i: ops.attention_prefill(out, q, k_pages, v_pages, table, request, positions, token0, count,
                                                                nq, 1 / math.sqrt(d), args.window, size, before + tokens,
                                                                splits, part_o, part_ml), args.repeats)
                print(f"attention_prefill tokens={tokens} after={before} group={size} splits={splits}: {seconds * 1e6:9.1f} us  "
                      f"{flops / seconds / 1e12:7.1f} TFLOP/s (keys a query may see)", flush=True)


def attention_decode(args) -> None:
    """One query token per request over `context` cached tokens."""
    nq, nkv, d, page, context = args.heads, args.kv_heads, args.head_dim, args.page_size, args.context
    for batch in _ints(args.batch):
        pages = batch * (context // page + 1)
        cache_bytes = batch * context * nkv * d * 2 * 2
        sets = max(1, min(8, int(3e9 / (pages * nkv * page * d * 2 * 2))))
        caches = [(torch.randn(pages + 1, nkv, page, d, device="cuda", dtype=torch.bfloat16),
                   torch.randn(pages + 1, nkv, d, page, device="cuda", dtype=torch.bfloat16)) for _ in range(sets)]
        table = torch.randperm(pages, device="cuda").to(torch.int32).view(batch, -1)
        q = torch.randn(batch, (nq + 2 * nkv) * d, device="cuda", dtype=torch.bfloat16)
        out = torch.empty(batch, nq * d, device="cuda", dtype=torch.bfloat16)
        request = torch.arange(batch, dtype=torch.int32, device="cuda")
        positions = torch.full((batch,), context - 1, dtype=torch.int32, device="cuda")
        for form in _ints(args.form):
            for splits in _ints(args.splits):
                part_o = torch.empty(batch, nq * splits * d, device="cuda")
                part_ml = torch.empty(batch, nq * splits * 2, device="cuda")
                seconds = _time(lambda i: ops.attention_decode(out, q, caches[i % sets][0], caches[i % sets][1], table, request, positions,
                                                               nq, 1 / math.sqrt(d), args.window, splits, part_o, part_ml, context,
                                                               form=form), args.repeats)
                print(f"attention_decode batch={batch} context={context} form={form} splits={splits}: {seconds * 1e6:8.1f} us  "
                      f"{cache_bytes / seconds / 1e9:7.0f} GB/s of cache", flush=True)


def gemm(args) -> None:
    """x [rows, K] times W[N, K]^T for the products of one layer: this package's kernel and torch.mm."""
    hidden, inter = args.hidden_size, args.intermediate_size
    qkv = (args.heads + 2 * args.kv_heads) * args.head_dim
    shapes = [("qkv", qkv, hidden), ("o", hidden, args.heads * args.head_dim), ("gate_up", 2 * inter, hidden), ("down", hidden, inter)]
    if args.vocab_size:
        shapes.append(("lm_head", args.vocab_size, hidden))
    # the few-rows kernel is timed up to its own limit, not the one steps use
    base = dict(few_rows_max=ops.few_rows_capacity(), whole_lines=not args.fragment_loads)
    if True:
        for name, n, k in shapes:
            sets = max(2, min(16, int(1.2e9 / (n * k * 2))))
            weights = [torch.randn(n, k, device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
            for rows in _ints(args.rows):
                x = torch.randn(rows, k, device="cuda", dtype=torch.bfloat16)
                out = torch.empty(rows, n, device="cuda", dtype=torch.bfloat16)
                variants = [("own", 0, 0), ("library", 0, 0), ("torch.mm", 0, 0)]
                if args.mid_sweep and 16 < rows <= 128:
                    # every shape with the plain deal of the weight rows; "even": dealt evenly where the shape allows
                    variants = [(f"mid w{wv} s{sp}", wv, sp) for wv in (4, 5, 6, 8) for sp in _ints(args.mid_sweep)] + [("mid even", 0, 0)] + variants
                for which, wv, sp in variants:
                    if which == "library":
                        call = lambda i: ops.library_gemm(out, x, weights[i % sets])
                    elif which == "torch.mm":
                        call = lambda i: torch.mm(x, weights[i % sets].t(), out=out)
                    else:
                        choice = ops.KernelChoice(mid_waves=wv, mid_splits=sp, mid_even=2 if which == "mid even" else 1 if which.startswith("mid") else 0, **base)
                        call = lambda i: ops.gemm(out, x, weights[i % sets], choice=choice)
                    note = ""
                    if which in ("own", "mid even") and 16 < rows <= 128 and k % 256 == 0:
                        note = "  %d waves x %d splits, %d workgroups, %d with a tile more" % ops.gemm_mid_deal(rows, n, k, choice)
                    seconds = _time(call, max(args.repeats, 2 * sets))
                    print(f"gemm {name:8s} rows={rows:5d} {which:10s} {seconds * 1e6:9.1f} us  {n * k * 2 / seconds / 1e9:8.0f} GB/s of weights  "
                          f"{2 * rows * n * k / seconds / 1e12:8.1f} TFLOP/s{note}", flush=True)
            del weights


def memory(args) -> None:
    """The rate at which a plain kernel streams memory once: what 'reads from memory' can mean on this GPU."""
    for megabytes in _ints(args.megabytes):
        buffers = [torch.randint(0, 1 << 30, (megabytes << 18,), dtype=torch.int32, device="cuda") for _ in range(max(2, min(6, 3072 // megabytes)))]
        for blocks in _ints(args.blocks):
            sink = torch.zeros(blocks, dtype=torch.int32, device="cuda")
            seconds = _time(lambda i: ops.stream_read(buffers[i % len(buffers)], sink, blocks), args.repeats)
            print(f"memory read {megabytes:5d} MB with {blocks:5d} workgroups: {seconds * 1e6:9.1f} us  {(megabytes << 20) / seconds / 1e9:7.0f} GB/s", flush=True)
        del buffers


def sampling(args) -> None:
    """Filtering the logits of a step (top-k, top-p, both) and choosing its tokens (greedy, drawn)."""
    vocab = args.vocab_size or 151936
    generator = torch.Generator().manual_seed(0)
    for rows in _ints(args.batch):
        base = (torch.randn(rows, vocab, generator=generator) * 3).cuda()
        copies = [base.clone() for _ in range(8)]
        temperature = torch.full((rows,), 0.8, device="cuda")
        seeds = torch.arange(rows, dtype=torch.int64, device="cuda")
        counters = torch.zeros(rows, dtype=torch.int32, device="cuda")
        out = torch.zeros(rows, dtype=torch.int32, device="cuda")
        for name, k, p in (("top_k 50", 50, 1.0), ("top_p 0.9", 0, 0.9), ("top_k 50, top_p 0.9", 50, 0.9)):
            top_k = torch.full((rows,), k, dtype=torch.int32, device="cuda")
            top_p = torch.full((rows,), p, device="cuda")

            def call(i):
                copies[i % 8].copy_(base)             # the filter writes into the logits: a fresh copy every time
                ops.filter_logits(copies[i % 8], temperature, top_k, top_p)

            copy_only = _time(lambda i: copies[i % 8].copy_(base), args.repeats)
            seconds = _time(call, args.repeats) - copy_only
            print(f"sampling rows={rows:3d} vocab={vocab} filter_logits {name:20s} {seconds * 1e6:8.1f} us", flush=True)
        for name, drawn in (("greedy", False), ("drawn", True)):
            seconds = _time(lambda i: ops.choose_tokens(out, base, *((temperature, seeds, counters) if drawn else ())), args.repeats)
            print(f"sampling rows={rows:3d} vocab={vocab} choose_tokens {name:20s} {seconds * 1e6:8.1f} us", flush=True)


def lds(args) -> None:
    """16-byte LDS reads in the shape of a matrix-core fragment (a lane's row is lane % 16, its piece lane / 16)
    for every distance between rows: what the layout of a tile in LDS has to respect."""
    units, iters = ops.compute_units(), 4096
    sink = torch.zeros(256, dtype=torch.int32, device="cuda")
    for stride in range(64, 321, 16):
        seconds = _time(lambda i: ops.probe_lds(sink, 2 * units, iters, stride), 5)
        per_cycle = 2 * 256 * iters * 8 * 16 / seconds / 2.4e9
        print(f"lds rows {stride:3d} bytes apart: {seconds * 1e3:7.3f} ms  {per_cycle:6.1f} bytes a cycle and compute unit (at 2.4 GHz)", flush=True)


def lines(args) -> None:
    """What one compute unit, and many, stream from memory with 16-byte loads, by the lines that 16 neighbouring
    lanes touch: 16 (the order of a matrix-core fragment: a lane's row is lane % 16), 2 (whole lines) or 4 (64
    bytes of a row to four neighbouring lanes)."""
    data = torch.randint(0, 1 << 30, (2048 << 18,), dtype=torch.int32, device="cuda")      # 2 GB, walked region by region: no call finds its bytes in a cache
    sink = torch.zeros(256, dtype=torch.int32, device="cuda")
    names = ("fragment order", "whole lines", "a row to four lanes")
    for blocks in _ints(args.blocks):
        for threads in (256, 1024):
            for kilobytes in (256, 1024):
                span = blocks * (kilobytes << 8)                                            # int32 elements a call
                regions = data.numel() // span
                for pattern in range(3):
                    seconds = _time(lambda i: ops.probe_lines(data[(i % regions) * span:(i % regions + 1) * span], sink, blocks, threads, kilobytes << 10, pattern),
                                    args.repeats)
                    print(f"lines {blocks:4d} workgroups of {threads:4d} threads, {kilobytes:4d} KB each, {names[pattern]:20s}: {seconds * 1e6:7.1f} us  "
                          f"{(kilobytes << 10) / seconds / 1e9:6.1f} GB/s a workgroup  {blocks * (kilobytes << 10) / seconds / 1e9:7.0f} GB/s", flush=True)


def mfma(args) -> None:
    """What the matrix cores sustain alone and with vector instructions of the same wave between the products."""
    units, iters = ops.compute_units(), 4000
    sink = torch.zeros(256, dtype=torch.float32, device="cuda")
    for valu, exps in ((0, False), (1, False), (2, False), (3, False), (4, False), (6, False), (2, True), (3, True)):
        seconds = _time(lambda i: ops.probe_mfma(sink, 8 * units, iters, valu, exps), 3)
        rate = 8 * units * 4 * iters * 32 * 16384 / seconds / 1e12
        print(f"mfma 16x16x32 bf16 with {valu} multiply-adds after each{' and an exponential after every second' if exps else ''}: "
              f"{seconds * 1e3:7.3f} ms  {rate:7.1f} TFLOP/s", flush=True)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="python -m llm_runtime_study_amd.kernels.microbench", description=__doc__.split("\n\n")[0])
    parser.add_argument("kernel", choices=["attention_prefill", "attention_decode", "gemm", "memory", "sampling", "lds", "mfma", "lines"])
    parser.add_argument("--heads", type=int, default=32)
    parser.add_argument("--kv-heads", type=int, default=8)
    parser.add_argument("--head-dim", type=int, default=128)
    parser.add_argument("--hidden-size", type=int, default=4096)
    parser.add_argument("--intermediate-size", type=int, default=12288)
    parser.add_argument("--vocab-size", type=int, default=0, help="gemm: also the LM head of this many rows; sampling: the vocabulary (default 151936)")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--window", type=int, default=0)
    parser.add_argument("--tokens", default="2048", help="attention_prefill: prompt lengths, comma separated")
    parser.add_argument("--before", type=int, default=0, help="attention_prefill: tokens of the request already in the cache (the queries are a later portion)")
    parser.add_argument("--key-splits", default="1", help="attention_prefill: workgroups per query group")
    parser.add_argument("--group", default="", help="attention_prefill: query group sizes (default: what the engine would choose)")
    parser.add_argument("--batch", default="1,8,64", help="attention_decode, sampling: batch sizes")
    parser.add_argument("--context", type=int, default=2048, help="attention_decode: cached tokens per request")
    parser.add_argument("--splits", default="1,2,4,8,16", help="attention_decode: workgroups per (token, kv head)")
    parser.add_argument("--form", default="0,1,2", help="attention_decode: 0 four waves, 1 four waves with the next tile on the way, 2 eight waves likewise")
    parser.add_argument("--rows", default="1,8,16,64,2048", help="gemm: numbers of rows")
    parser.add_argument("--fragment-loads", action="store_true", help="gemm: the few-rows kernel loads weights and activations as MFMA fragments (64 bytes of 16 rows), not as whole lines")
    parser.add_argument("--mid-sweep", default="", help="gemm: also time the kernel for 17..128 rows with 4, 5, 6 and 8 waves at these numbers of K splits, and with its rows dealt evenly")
    parser.add_argument("--megabytes", default="32,200,1200", help="memory: sizes of the buffers read")
    parser.add_argument("--blocks", default="512,2048,8192", help="memory, lines: numbers of workgroups (lines: try 8,64,256,512)")
    parser.add_argument("--repeats", type=int, default=20)
    args = parser.parse_args(argv)
    if not torch.cuda.is_available():
        print("microbench needs the GPU", file=sys.stderr)
        return 2
    ops.library()
    {"attention_prefill": attention_prefill, "attention_decode": attention_decode, "gemm": gemm, "memory": memory, "sampling": sampling, "lds": lds,
     "mfma": mfma, "lines": lines}[args.kernel](args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
