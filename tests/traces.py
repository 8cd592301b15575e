"""Builders of replay traces (the JSON steps that bin/trace_run reads) and the comparison
of what a replay wrote with the plain implementation's whole-sequence logits."""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch


def whole(requests: dict) -> list[dict]:
    """Each request alone and whole: one step per request, logits at every position."""
    steps = []
    for step, (key, tokens) in enumerate(requests.items()):
        steps.append({"step": step, "entries": [{"id": key, "tokens": list(tokens), "want": list(range(len(tokens)))}], "end": [key]})
    return steps


def prefill_then_decode(requests: dict, tail: int = 32) -> list[dict]:
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps, step = [], 0
    for key, tokens in requests.items():
        tokens = list(tokens)
        head = max(1, len(tokens) - tail)
        steps.append({"step": step, "entries": [{"id": key, "tokens": tokens[:head], "want": list(range(head))}], "end": []})
        step += 1
        for i in range(head, len(tokens)):
            steps.append({"step": step, "entries": [{"id": key, "tokens": [tokens[i]], "want": [0]}],
                          "end": [key] if i == len(tokens) - 1 else []})
            step += 1
        if head == len(tokens):
            steps[-1]["end"] = [key]
    return steps


def portions(requests: dict, sizes=(7, 16, 2, 5, 3, 2, 33, 2, 17, 1, 4)) -> list[dict]:
    """Each request alone, cut into portions of changing size, down to two tokens."""
    steps, step = [], 0
    for key, tokens in requests.items():
        tokens, at, turn = list(tokens), 0, 0
        while at < len(tokens):
            n = min(sizes[turn % len(sizes)], len(tokens) - at)
            turn += 1
            steps.append({"step": step, "entries": [{"id": key, "tokens": tokens[at:at + n], "want": list(range(n))}],
                          "end": [key] if at + n == len(tokens) else []})
            at += n
            step += 1
    return steps


def mixed(requests: dict, seed: int = 0, max_live: int = 4, max_tokens: int | None = None, round_to: int = 64) -> tuple[list[dict], int]:
    """Up to `max_live` requests live at once: portions of some beside single tokens of others,
    requests pausing for a step now and then, new ones admitted as old ones end, so that the
    pages a finished request gave back are used again.  Returns the steps and the largest number
    of tokens (each request rounded up to `round_to`) that live requests held at any time."""
    rng = np.random.default_rng(seed)
    waiting = [(k, list(t)) for k, t in requests.items()]
    live: dict = {}
    steps, step, peak = [], 0, 0

    def held(extra=None):
        total = 0
        for k, (toks, at) in live.items():
            n = at + (extra.get(k, 0) if extra else 0)
            total += -(-max(n, 1) // round_to) * round_to
        return total

    while waiting or live:
        while waiting and len(live) < max_live:
            key, toks = waiting[0]
            need = -(-len(toks) // round_to) * round_to
            if max_tokens is not None and live and sum(-(-len(t) // round_to) * round_to for t, _ in live.values()) + need > max_tokens:
                break
            waiting.pop(0)
            live[key] = (toks, 0)
        entries, ends = [], []
        for key in list(live):
            toks, at = live[key]
            if len(live) > 1 and rng.random() < 0.15:
                continue  # sits this step out
            left = len(toks) - at
            kind = rng.random()
            if kind < 0.45:
                n = 1
            elif kind < 0.6:
                n = 2
            else:
                n = int(rng.integers(2, 40))
            n = min(n, left)
            want = sorted(set(rng.choice(n, size=min(n, int(rng.integers(1, 4))), replace=False).tolist() + [n - 1]))
            entries.append({"id": key, "tokens": toks[at:at + n], "want": want, "_at": at})
            live[key] = (toks, at + n)
            if at + n == len(toks):
                ends.append(key)
        peak = max(peak, held())
        if entries:
            steps.append({"step": step, "entries": entries, "end": ends})
            step += 1
        for key in ends:
            del live[key]
    return steps, peak


def strip(steps: list[dict]) -> str:
    """JSON lines without the bookkeeping keys."""
    lines = []
    for s in steps:
        clean = {"step": s["step"], "entries": [{k: v for k, v in e.items() if not k.startswith("_")} for e in s["entries"]], "end": s["end"]}
        lines.append(json.dumps(clean))
    return "\n".join(lines) + "\n"


def collect(steps: list[dict], out_dir: Path, vocab: int) -> dict:
    """{request id: {position: logits row}} from the files a replay wrote."""
    got: dict = {}
    progress: dict = {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = Path(out_dir) / f"{s['step']}.f32"
        if wanted == 0:
            assert not path.exists()
            for e in s["entries"]:
                progress[e["id"]] = progress.get(e["id"], 0) + len(e["tokens"])
            continue
        data = np.fromfile(path, dtype="<f4")
        assert data.size == wanted * vocab, f"step {s['step']}: {data.size} floats for {wanted} rows of {vocab}"
        data = data.reshape(wanted, vocab)
        row = 0
        for e in s["entries"]:
            at = progress.get(e["id"], 0)
            for place in e["want"]:
                got.setdefault(e["id"], {})[at + place] = torch.from_numpy(data[row].copy())
                row += 1
            progress[e["id"]] = at + len(e["tokens"])
    return got
