"""Continuous batching with chunked prefill above the step function.

Every step() builds one mixed batch under a token budget and runs it as one call of the
step function:

  1. admission, first come first served: the head of the queue is admitted while a batch
     slot is free and the cache can promise pages for its whole lifetime (prompt + output
     limit); nothing jumps the queue.  A prompt that leaves no room for output ends at once
     with `context_length`, without a slot or a forward.
  2. every running request that has finished its prompt contributes its last sampled token;
  3. the rest of the budget goes to prompt portions, oldest request first, cut wherever the
     budget ends; a request asks for logits only in the step that holds its last prompt token;
  4. one token is sampled for every row that asked for logits; a request that finishes
     (eos, then max_new_tokens or context_length) gives its pages and slot back at once.

Pages cannot run out in the middle of a request: admission reserves the lifetime, so when
the pool is short the head of the queue waits until running requests finish.  A request that
could never fit is refused when it is added.  Any failure aborts every request, frees every
page and re-raises.

Reference mini_llm/generation.py:112-399 (same admission, finish and failure rules; it
prefills whole prompts alone at admission, here prompts are cut under `max_step_tokens` and
share steps with decoding requests).
"""

from __future__ import annotations

import itertools
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Sequence

from ..errors import GenerationError, SamplingError
from ..sampling import SamplingConfig, SamplingRow, request_seed
from ..text import ChatMessage, TextStream
from .step import StepEntry


@dataclass(frozen=True)
class GenerationEvent:
    """One streamed token and the text so far (reference mini_llm/generation.py:34-44)."""

    token_id: int | None
    token_index: int | None
    text_delta: str
    text: str
    finish_reason: str | None = None   # "eos" | "max_new_tokens" | "context_length"
    model_seconds: float | None = None
    prompt_token_count: int | None = None


@dataclass
class _Waiting:
    index: int
    prompt: list[int]
    output_limit: int
    max_new_tokens: int
    sampling: SamplingConfig


@dataclass
class _Running:
    index: int
    prompt: list[int]
    output_limit: int
    max_new_tokens: int
    sampling: SamplingConfig
    seed: int
    cache: object
    decoder: TextStream
    fed: int = 0                      # prompt tokens already run
    produced: int = 0                 # tokens sampled so far
    next_token: int | None = None     # sampled, not yet run
    tokens: list = field(default_factory=list)


class BatchScheduler:
    def __init__(self, runner, sampler, *, max_batch_size: int, max_seq_len: int, max_step_tokens: int,
                 eos_token_ids: Sequence[int] = (), vocab_size: int | None = None, tokenizer=None,
                 synchronize: Callable[[], None] | None = None, decode_steps_per_launch: int = 1, launch_ahead: bool = False):
        if max_batch_size <= 0:
            raise GenerationError("max_batch_size must be positive")
        if max_seq_len <= 0 or max_seq_len > runner.cache.max_seq_len:
            raise GenerationError(f"max_seq_len must be within [1, {runner.cache.max_seq_len}], got {max_seq_len}")
        if max_step_tokens < max_batch_size:
            raise GenerationError(
                f"the token budget of a step ({max_step_tokens}) must hold one token of each of the {max_batch_size} batch slots")
        self.runner, self.sampler, self.tokenizer = runner, sampler, tokenizer
        self.cache = runner.cache
        self.max_batch_size, self.context_limit, self.max_step_tokens = max_batch_size, max_seq_len, max_step_tokens
        self.vocab_size = vocab_size
        self._eos = frozenset(eos_token_ids)
        self._synchronize = synchronize
        if decode_steps_per_launch < 1:
            raise GenerationError(f"decode_steps_per_launch must be at least 1, got {decode_steps_per_launch}")
        # When every running request decodes, up to this many steps run from one launch (the step
        # function chooses each token and feeds it back in on the device): the host, which needs
        # about a tenth of a millisecond between steps, is then out of the loop.  Tokens a request
        # produced after its end-of-sequence token are dropped; a waiting request is admitted up
        # to that many steps later than it could have been.
        self.decode_steps_per_launch = decode_steps_per_launch
        # launch_ahead: while every running request decodes, the next launch of decode steps is queued before the tokens
        # of the one before are read, so the device goes from launch to launch without waiting for the host (which
        # reads tokens, finishes requests and streams text meanwhile).  The tokens of a launch then come out of the
        # step() call after the one that queued it.  A request that ends in a launch (its end-of-sequence token) has
        # run on in the launch queued behind it; those tokens are dropped like the ones after an end-of-sequence
        # token inside one launch, and a waiting request is admitted that much later.
        self.launch_ahead = launch_ahead and decode_steps_per_launch > 1 and hasattr(runner, "decode_launch_begin")
        self._in_flight = None          # (launch, the requests of its rows, when it was queued)
        self._collected_at = 0.0
        self._ids = itertools.count()
        self._waiting: deque[_Waiting] = deque()
        self._running: list[_Running] = []
        self.step_log: list[list[tuple[int, int]]] = []   # per step: (request index, tokens run)

    # ---------------------------------------------------------------- requests
    def add_request(self, prompt, *, max_new_tokens: int, sampling: SamplingConfig = SamplingConfig(),
                    enable_thinking: bool = False) -> int:
        """Queue one request; `prompt` is a list of token ids or of ChatMessage.  Returns its index."""
        if max_new_tokens <= 0:
            raise GenerationError("max_new_tokens must be positive")
        if self.vocab_size is not None and sampling.top_k is not None and sampling.top_k > self.vocab_size:
            raise SamplingError(f"top_k {sampling.top_k} exceeds vocabulary size {self.vocab_size}")
        prompt_ids = self._token_ids(prompt, enable_thinking)
        length = len(prompt_ids)
        if length == 0:
            raise GenerationError("a prompt needs at least one token")
        if length > self.context_limit:
            raise GenerationError(f"prompt has {length} tokens but model context limit is {self.context_limit}")
        output_limit = min(max_new_tokens, self.context_limit - length)
        required = length + output_limit
        if output_limit > 0 and required > self.cache.capacity:
            raise GenerationError(f"request needs {required} cache tokens but the KV cache holds {self.cache.capacity}")
        index = next(self._ids)
        self._waiting.append(_Waiting(index, prompt_ids, output_limit, max_new_tokens, sampling))
        return index

    def _token_ids(self, prompt, enable_thinking: bool) -> list[int]:
        if isinstance(prompt, (list, tuple)) and all(isinstance(t, int) and not isinstance(t, bool) for t in prompt):
            ids = list(prompt)
            if self.vocab_size is not None and any(not 0 <= t < self.vocab_size for t in ids):
                raise GenerationError(f"input_ids must be within vocabulary [0, {self.vocab_size})")
            return ids
        if isinstance(prompt, (list, tuple)) and all(isinstance(m, ChatMessage) for m in prompt):
            if self.tokenizer is None:
                raise GenerationError("a text prompt needs a tokenizer; this model folder has none (pass token ids)")
            return self.tokenizer.encode(self.tokenizer.format_chat(prompt, enable_thinking=enable_thinking))
        raise GenerationError("a prompt must be a list of token ids or of ChatMessage")

    @property
    def has_unfinished(self) -> bool:
        return bool(self._waiting or self._running)

    @property
    def steps_in_flight(self) -> int:
        """Decode steps of the launch that has been queued and whose tokens the next step() call returns (0: none)."""
        return 0 if self._in_flight is None else self._in_flight[0].steps

    @property
    def num_waiting(self) -> int:
        return len(self._waiting)

    @property
    def num_running(self) -> int:
        return len(self._running)

    # -------------------------------------------------------------------- step
    def step(self) -> list[tuple[int, GenerationEvent]]:
        """Admit, run one mixed batch, sample; returns (request index, event) pairs."""
        events: list[tuple[int, GenerationEvent]] = []
        try:
            if self._in_flight is not None:
                self._collect(events)
                return events
            self._admit(events)
            steps = self._decode_steps_ahead()
            if steps > 1 and self.launch_ahead:
                self._queue_launch(steps, None)
                self._collect(events)
                return events
            if steps > 1:
                self._decode_several(steps, events)
                return events
            entries, rows = self._build_batch()
            if entries:
                started = self._now()
                logits = self.runner.step(entries)
                tokens = self.sampler.choose(logits, [row for _, row in rows]) if rows else []
                # reading the tokens has waited for the step; a step that samples nothing stays in flight
                seconds = self._now(wait=False) - started if started is not None and rows else None
                self._finish_step(rows, tokens, seconds, events)
        except BaseException:       # an interrupt from the keyboard frees everything as well
            self.abort_all()
            raise
        return events

    # ------------------------------------------------------ launches queued ahead
    def _queue_launch(self, steps: int, after) -> None:
        """Queue a launch of decode steps of every running request; `after`: (launch, requests, ...) it follows directly."""
        running = list(self._running) if after is None else after[1]
        entries = [StepEntry(r.cache, [r.next_token if r.next_token is not None else 0], [0]) for r in running]
        rows = [SamplingRow(r.sampling, r.seed, r.produced) for r in running] if after is None else None
        if after is not None and after[0].sampled:
            rows = [SamplingRow(r.sampling, r.seed, r.produced + after[0].steps) for r in running]
        launch = self.runner.decode_launch_begin(entries, steps, rows, after=None if after is None else after[0])
        self._in_flight = (launch, running, time.perf_counter())

    def _collect(self, events) -> None:
        """The tokens of the launch in flight.  Before they are waited for, the launch after it is queued if no
        request can reach its length limit inside the one in flight and nothing waits that could be admitted now."""
        launch, running, queued_at = self._in_flight
        following = None
        still = {id(r) for r in self._running}
        left = min(r.output_limit - r.produced for r in running) - launch.steps
        # (a launch can only be followed by one of the same requests: once one of them has ended, the launch in flight
        # is the last of its chain, and the next step starts anew with those that are left)
        if self.launch_ahead and left >= 1 and all(id(r) in still for r in running) and not self._could_admit():
            self._queue_launch(min(self.decode_steps_per_launch, left), self._in_flight)
            following = self._in_flight
        self._in_flight = None
        try:
            chosen = self.runner.decode_launch_end(launch)
        except BaseException:
            if following is not None:
                self.runner.decode_launch_drop(following[0])
            raise
        now = time.perf_counter()
        seconds = (now - max(queued_at, self._collected_at)) / launch.steps if self._synchronize is not None else None
        self._collected_at = now                                 # a launch queued behind another began when that one's tokens were due
        alive = [r for r in running if id(r) in still]           # a request that ended in the launch before is not looked at again
        for tokens in chosen:
            if not alive:
                break
            by_request = dict(zip(map(id, running), tokens))
            self.step_log.append([(r.index, 1) for r in alive])
            self._finish_step([(r, None) for r in alive], [by_request[id(r)] for r in alive], seconds, events)
            still = {id(r) for r in self._running}
            alive = [r for r in alive if id(r) in still]
        if following is not None:
            if alive:
                self._in_flight = following
            else:
                self.runner.decode_launch_drop(following[0])     # every one of its requests has ended: nobody wants its tokens

    def _could_admit(self) -> bool:
        """Whether the head of the queue could be admitted right now (then decoding pauses for a step that takes it in)."""
        if not self._waiting:
            return False
        head = self._waiting[0]
        if head.output_limit == 0:
            return True
        lifetime = len(head.prompt) + head.output_limit
        return len(self._running) < self.max_batch_size and self.cache.can_admit(lifetime, self.max_step_tokens)

    def _now(self, wait: bool = True):
        """The clock for `model_seconds` (None if the scheduler was given no way to wait for the device).  wait: after
        everything queued on the device has finished, so that the time of a step is its own."""
        if self._synchronize is None:
            return None
        if wait:
            self._synchronize()
        return time.perf_counter()

    def abort_all(self) -> None:
        """Release every running request's cache and drop every waiting request."""
        in_flight, self._in_flight = self._in_flight, None
        if in_flight is not None:
            self.runner.decode_launch_drop(in_flight[0])
        running, self._running = self._running, []
        self._waiting.clear()
        for request in running:
            self.cache.release(request.cache)

    def _admit(self, events) -> None:
        while self._waiting:
            head = self._waiting[0]
            if head.output_limit == 0:
                self._waiting.popleft()
                events.append((head.index, GenerationEvent(None, None, "", "", "context_length", None, len(head.prompt))))
                continue
            lifetime = len(head.prompt) + head.output_limit
            if len(self._running) >= self.max_batch_size or not self.cache.can_admit(lifetime, self.max_step_tokens):
                return
            self._waiting.popleft()
            cache = self.cache.admit(head.index, reserve_tokens=lifetime, max_step_tokens=self.max_step_tokens)
            self._running.append(_Running(head.index, head.prompt, head.output_limit, head.max_new_tokens, head.sampling,
                                          request_seed(head.sampling), cache, TextStream(self.tokenizer)))

    def _build_batch(self):
        budget = self.max_step_tokens
        entries, rows, log = [], [], []
        for request in self._running:          # decoding requests first: one token each
            if request.next_token is not None:
                entries.append(StepEntry(request.cache, [request.next_token], [0]))
                rows.append((request, SamplingRow(request.sampling, request.seed, request.produced)))
                log.append((request.index, 1))
                budget -= 1
        for request in self._running:          # then prompt portions, oldest first
            if request.next_token is None and budget > 0:
                n = min(len(request.prompt) - request.fed, budget)
                last = request.fed + n == len(request.prompt)
                entries.append(StepEntry(request.cache, request.prompt[request.fed:request.fed + n], [n - 1] if last else []))
                if last:
                    rows.append((request, SamplingRow(request.sampling, request.seed, request.produced)))
                request.fed += n
                log.append((request.index, n))
                budget -= n
        if log:
            self.step_log.append(log)
        return entries, rows

    def _decode_steps_ahead(self) -> int:
        """How many decode steps the next launch may hold: more than one only if every running request
        is decoding and the step function can choose tokens and feed them back in by itself (all
        greedy, unless it also samples); never more than any request has left to produce."""
        if self.decode_steps_per_launch <= 1 or not self._running or not hasattr(self.runner, "decode_steps"):
            return 1
        if any(r.next_token is None for r in self._running):
            return 1
        if not getattr(self.runner, "decode_steps_sample", False) and any(not r.sampling.greedy for r in self._running):
            return 1
        steps = min(self.decode_steps_per_launch, min(r.output_limit - r.produced for r in self._running))
        if steps <= 1:
            return 1
        entries = [StepEntry(r.cache, [r.next_token], [0]) for r in self._running]
        return steps if self.runner.can_decode_steps(entries) else 1

    def _decode_several(self, steps: int, events) -> None:
        running = list(self._running)
        entries = [StepEntry(r.cache, [r.next_token], [0]) for r in running]
        started = self._now()
        if getattr(self.runner, "decode_steps_sample", False):
            chosen = self.runner.decode_steps(entries, steps, [SamplingRow(r.sampling, r.seed, r.produced) for r in running])
        else:
            chosen = self.runner.decode_steps(entries, steps)
        seconds = (self._now(wait=False) - started) / steps if started is not None else None     # the tokens are back: the launch has finished
        alive = running
        for tokens in chosen:
            if not alive:
                break
            by_request = dict(zip(map(id, running), tokens))
            self.step_log.append([(r.index, 1) for r in alive])
            rows = [(r, None) for r in alive]
            self._finish_step(rows, [by_request[id(r)] for r in alive], seconds, events)
            still = {id(r) for r in self._running}
            alive = [r for r in alive if id(r) in still]

    def _finish_step(self, rows, tokens, seconds, events) -> None:
        finished = set()
        for (request, _), token in zip(rows, tokens):
            delta = request.decoder.push(token)
            request.produced += 1
            request.tokens.append(token)
            reason = None
            if token in self._eos:
                reason = "eos"
            elif request.produced == request.output_limit:
                reason = "context_length" if request.output_limit < request.max_new_tokens else "max_new_tokens"
            events.append((request.index, GenerationEvent(
                token, request.produced - 1, delta, request.decoder.text, reason, seconds,
                len(request.prompt) if request.produced == 1 else None)))
            if reason is None:
                request.next_token = token
            else:
                self.cache.release(request.cache)
                finished.add(id(request))
        if finished:
            self._running = [r for r in self._running if id(r) not in finished]


def generate(scheduler: BatchScheduler, prompts, *, max_new_tokens: int, sampling: SamplingConfig = SamplingConfig(),
             enable_thinking: bool = False):
    """Queue `prompts` and iterate over their events until all are finished
    (reference mini_llm/generation.py:402-450); closing the iterator frees everything."""
    if not prompts:
        raise GenerationError("a generation batch must contain at least one request")
    for prompt in prompts:
        scheduler.add_request(prompt, max_new_tokens=max_new_tokens, sampling=sampling, enable_thinking=enable_thinking)

    def iterate():
        try:
            while scheduler.has_unfinished:
                yield from scheduler.step()
        finally:
            scheduler.abort_all()

    return iterate()
