"""Scheduler decisions with a fake step function: admission, portions under the token budget,
decoding, finishing, freeing, waiting for pages, failure (CPU)."""

import pytest
import torch

from llm_runtime_study_amd.cache import CacheManager
from llm_runtime_study_amd.engine.scheduler import BatchScheduler, generate
from llm_runtime_study_amd.errors import GenerationError, KVCacheError, SamplingError
from llm_runtime_study_amd.parts import PagedKVNeed
from llm_runtime_study_amd.sampling import SamplingConfig

VOCAB = 50


class FakeRunner:
    """Extends caches like the real step function and returns logits that make request i's
    k-th token equal `script[i][k]`; the request is known by its cache's request_id."""

    def __init__(self, script, num_pages=16, page_size=4, max_requests=4, max_seq_len=64):
        self.cache = CacheManager([PagedKVNeed(1, 8)], page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                                  max_seq_len=max_seq_len, dtype=torch.float32, device="cpu", allocate_storage=False)
        self.script, self.produced, self.calls, self.fail_at = script, {}, [], None

    def step(self, entries):
        if self.fail_at is not None and len(self.calls) == self.fail_at:
            raise RuntimeError("injected failure")
        self.calls.append([(e.cache.request_id, list(e.tokens), list(e.want)) for e in entries])
        rows = []
        for e in entries:
            self.cache.extend(e.cache, len(e.tokens))
            for _ in e.want:
                k = self.produced.get(e.cache.request_id, 0)
                self.produced[e.cache.request_id] = k + 1
                row = torch.zeros(VOCAB)
                row[self.script[e.cache.request_id][k]] = 1.0
                rows.append(row)
        self.cache.check_invariants()
        return torch.stack(rows) if rows else None


class FakeSampler:
    def choose(self, logits, rows):
        assert logits.shape[0] == len(rows)
        return logits.argmax(-1).tolist()


def scheduler(runner, **options):
    defaults = dict(max_batch_size=2, max_seq_len=64, max_step_tokens=8, eos_token_ids=(1,), vocab_size=VOCAB)
    defaults.update(options)
    return BatchScheduler(runner, FakeSampler(), **defaults)


def drain(s):
    events = []
    while s.has_unfinished:
        events += s.step()
    return events


def test_prompt_is_cut_under_the_budget_and_samples_only_on_its_last_portion():
    runner = FakeRunner({0: [7, 8, 1]})
    s = scheduler(runner, max_step_tokens=8)
    s.add_request(list(range(10, 30)), max_new_tokens=5)
    events = drain(s)
    assert [len(c[0][1]) for c in runner.calls] == [8, 8, 4, 1, 1]
    assert [c[0][2] for c in runner.calls] == [[], [], [3], [0], [0]]
    assert runner.calls[3][0][1] == [7] and runner.calls[4][0][1] == [8]
    assert [(i, e.token_id, e.token_index, e.finish_reason) for i, e in events] == [(0, 7, 0, None), (0, 8, 1, None), (0, 1, 2, "eos")]
    assert events[0][1].prompt_token_count == 20 and events[1][1].prompt_token_count is None
    assert runner.cache.used_pages() == 0 and runner.cache.active_requests == 0


def test_decodes_come_first_and_portions_share_the_step():
    runner = FakeRunner({0: [5, 6, 7, 8, 9, 9, 9], 1: [4, 4, 4, 4]})
    s = scheduler(runner, max_step_tokens=6, max_batch_size=2)
    s.add_request([2] * 3, max_new_tokens=6)
    s.add_request([3] * 11, max_new_tokens=3)
    drain(s)
    # (request, tokens run) per step: request 1's prompt fills what request 0 leaves of the budget
    assert s.step_log[:4] == [[(0, 3), (1, 3)], [(0, 1), (1, 5)], [(0, 1), (1, 3)], [(0, 1), (1, 1)]]
    first_mixed = runner.calls[1]
    assert first_mixed[0] == (0, [5], [0]) and first_mixed[1][2] == []   # decode row first, portion wants nothing yet


def test_finish_reasons_and_compaction():
    # reference tests/test_generation.py:387-400, 464-496
    runner = FakeRunner({0: [9, 9, 9], 1: [9, 1], 2: [9, 9, 9, 9]}, max_seq_len=8)
    s = scheduler(runner, max_batch_size=3, max_seq_len=8, max_step_tokens=16)
    s.add_request([2, 2], max_new_tokens=3)            # ends by max_new_tokens
    s.add_request([2, 2], max_new_tokens=5)            # ends by eos
    s.add_request([2] * 5, max_new_tokens=10)          # context clips the output to 3
    events = drain(s)
    last = {i: e for i, e in events}
    assert last[0].finish_reason == "max_new_tokens" and last[0].token_index == 2
    assert last[1].finish_reason == "eos" and last[1].token_index == 1
    assert last[2].finish_reason == "context_length" and last[2].token_index == 2
    # after request 1 ended, the decode batch holds the survivors in their old order
    assert [[r for r, _, _ in call] for call in runner.calls] == [[0, 1, 2], [0, 1, 2], [0, 2]]


def test_zero_room_prompt_ends_without_a_forward():
    runner = FakeRunner({1: [9]}, max_seq_len=8)
    s = scheduler(runner, max_seq_len=8)
    s.add_request([2] * 8, max_new_tokens=4)
    s.add_request([2] * 3, max_new_tokens=1)
    events = s.step()
    assert (events[0][0], events[0][1].finish_reason, events[0][1].token_id, events[0][1].prompt_token_count) == (0, "context_length", None, 8)
    assert events[1][0] == 1 and events[1][1].finish_reason == "max_new_tokens"
    assert len(runner.calls) == 1 and runner.calls[0][0][0] == 1


def test_requests_wait_for_a_slot_first_come_first_served():
    # reference tests/test_generation.py:515-550
    runner = FakeRunner({0: [9, 9, 9], 1: [9], 2: [9, 9]})
    s = scheduler(runner, max_batch_size=2)
    for n in (3, 1, 2):
        s.add_request([2, 2], max_new_tokens=n)
    s.step()
    assert (s.num_running, s.num_waiting) == (1, 1)   # request 1 finished at once, request 2 still waits
    s.step()
    assert (s.num_running, s.num_waiting) == (2, 0)
    drain(s)
    assert [[r for r, _, _ in call] for call in runner.calls] == [[0, 1], [0, 2], [0, 2]]


def test_head_of_queue_waits_for_pages_and_nothing_jumps_it():
    # pool of 6 pages of 4 tokens; reference tests/test_generation.py:552-568
    runner = FakeRunner({0: [9, 9, 9, 9], 1: [9, 9], 2: [9]}, num_pages=6)
    s = scheduler(runner, max_batch_size=3)
    s.add_request([2] * 12, max_new_tokens=4)     # lifetime 16 tokens = 4 pages
    s.add_request([2] * 10, max_new_tokens=2)     # 3 pages: does not fit beside request 0
    s.add_request([2] * 2, max_new_tokens=1)      # 1 page: would fit, but must not jump the queue
    s.step()
    assert (s.num_running, s.num_waiting) == (1, 2)
    events = drain(s)
    order = [i for i, e in events if e.prompt_token_count is not None]
    assert order == [0, 1, 2]
    first_step_of = {}
    for n, call in enumerate(runner.calls):
        for r, _, _ in call:
            first_step_of.setdefault(r, n)
    last_step_of_0 = max(n for n, call in enumerate(runner.calls) if any(r == 0 for r, _, _ in call))
    assert first_step_of[1] > last_step_of_0 and first_step_of[2] >= first_step_of[1]
    assert runner.cache.used_pages() == 0


def test_requests_that_can_never_run_are_refused_when_added():
    runner = FakeRunner({}, num_pages=4)      # 16 tokens of cache
    s = scheduler(runner, max_seq_len=32)
    with pytest.raises(GenerationError, match="max_new_tokens must be positive"):
        s.add_request([2], max_new_tokens=0)
    with pytest.raises(GenerationError, match="prompt has 33 tokens but model context limit is 32"):
        s.add_request([2] * 33, max_new_tokens=1)
    with pytest.raises(GenerationError, match="needs 20 cache tokens but the KV cache holds 16"):
        s.add_request([2] * 12, max_new_tokens=8)
    with pytest.raises(SamplingError, match="top_k 51 exceeds vocabulary size 50"):
        s.add_request([2], max_new_tokens=1, sampling=SamplingConfig(temperature=1.0, top_k=51))
    with pytest.raises(GenerationError, match="within vocabulary"):
        s.add_request([2, 50], max_new_tokens=1)
    with pytest.raises(GenerationError, match="needs a tokenizer"):
        from llm_runtime_study_amd import ChatMessage
        s.add_request([ChatMessage("user", "hi")], max_new_tokens=1)
    with pytest.raises(GenerationError, match="must hold one token of each"):
        scheduler(runner, max_batch_size=4, max_step_tokens=3)
    assert not s.has_unfinished


def test_failure_frees_every_request_and_reraises():
    # reference tests/test_generation.py:592-610
    runner = FakeRunner({0: [9] * 5, 1: [9] * 5})
    s = scheduler(runner)
    s.add_request([2] * 5, max_new_tokens=5)
    s.add_request([2] * 5, max_new_tokens=5)
    s.add_request([2] * 5, max_new_tokens=5)
    s.step()
    runner.fail_at = len(runner.calls)
    with pytest.raises(RuntimeError, match="injected failure"):
        s.step()
    assert not s.has_unfinished and runner.cache.used_pages() == 0 and runner.cache.active_requests == 0
    runner.cache.check_invariants()


def test_closing_the_iterator_frees_everything():
    runner = FakeRunner({0: [9] * 9})
    s = scheduler(runner)
    stream = generate(s, [[2, 2, 2]], max_new_tokens=9)
    assert next(stream)[1].token_id == 9
    assert runner.cache.used_pages() > 0
    stream.close()
    assert runner.cache.used_pages() == 0 and not s.has_unfinished
    with pytest.raises(GenerationError, match="at least one request"):
        generate(s, [], max_new_tokens=1)


def test_sampling_rows_carry_each_requests_own_seed_and_counter():
    seen = []

    class RecordingSampler(FakeSampler):
        def choose(self, logits, rows):
            seen.append([(r.seed, r.counter, r.config.temperature) for r in rows])
            return super().choose(logits, rows)

    runner = FakeRunner({0: [9, 9, 9], 1: [9, 9]})
    s = BatchScheduler(runner, RecordingSampler(), max_batch_size=2, max_seq_len=64, max_step_tokens=8, vocab_size=VOCAB)
    s.add_request([2, 2], max_new_tokens=3, sampling=SamplingConfig(temperature=0.8, seed=11))
    s.add_request([2, 2], max_new_tokens=2, sampling=SamplingConfig(temperature=0.5, seed=12))
    drain(s)
    assert seen == [[(11, 0, 0.8), (12, 0, 0.5)], [(11, 1, 0.8), (12, 1, 0.5)], [(11, 2, 0.8)]]


class SeveralStepsRunner(FakeRunner):
    """A fake step function that can also run several greedy decode steps from one call, as the real
    one does on the device: it extends every cache by that many tokens and reports what each step chose."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.launches, self.sampling_seen = [], []

    def can_decode_steps(self, entries):
        return all(len(e.tokens) == 1 for e in entries)

    def decode_steps(self, entries, steps, sampling=None):
        self.launches.append((steps, [e.cache.request_id for e in entries]))
        self.sampling_seen.append(None if sampling is None else [(row.config.temperature, row.seed, row.counter) for row in sampling])
        chosen = []
        for e in entries:
            self.cache.extend(e.cache, steps)
        for _ in range(steps):
            row = []
            for e in entries:
                k = self.produced.get(e.cache.request_id, 0)
                self.produced[e.cache.request_id] = k + 1
                script = self.script[e.cache.request_id]
                row.append(script[k] if k < len(script) else 0)
            chosen.append(row)
        self.cache.check_invariants()
        return chosen


def test_several_decode_steps_per_launch_give_the_same_events():
    script = {0: [7, 8, 9, 10, 11, 12, 13], 1: [20, 21, 1, 22, 23, 24, 25]}     # request 1 meets eos (1) as its third token

    def run(per_launch):
        runner = SeveralStepsRunner(script)
        s = scheduler(runner, decode_steps_per_launch=per_launch)
        s.add_request([3, 4, 5], max_new_tokens=7)
        s.add_request([6, 2], max_new_tokens=7)
        events = [(i, e.token_id, e.token_index, e.finish_reason) for i, e in drain(s)]
        assert runner.cache.active_requests == 0 and runner.cache.used_pages() == 0
        return events, runner, s

    single, _, log_single = run(1)
    several, runner, log_several = run(4)
    assert sorted(single) == sorted(several)
    assert [t for i, t, _, _ in several if i == 1] == [20, 21, 1]               # nothing after the end-of-sequence token
    assert [t for i, t, _, _ in several if i == 0] == [7, 8, 9, 10, 11, 12, 13]
    # prompts run as ordinary steps; then launches of 4 steps for both, and what is left for request 0 alone
    assert runner.launches == [(4, [0, 1]), (2, [0])]
    assert log_single.step_log == log_several.step_log


def test_several_decode_steps_need_greedy_requests_and_room():
    script = {0: [7, 8, 9, 10], 1: [20, 21, 22, 23]}
    runner = SeveralStepsRunner(script)
    s = scheduler(runner, decode_steps_per_launch=4)
    s.add_request([3, 4], max_new_tokens=4, sampling=SamplingConfig(temperature=0.7, seed=1))
    s.add_request([5], max_new_tokens=4)
    drain(s)
    assert runner.launches == []                                                # a sampled request keeps the host in the loop
    runner = SeveralStepsRunner(script)
    s = scheduler(runner, decode_steps_per_launch=8)
    s.add_request([3, 4], max_new_tokens=4)
    s.add_request([5], max_new_tokens=3)
    drain(s)
    assert runner.launches == [(2, [0, 1])]                                     # never more steps than the shortest has left
    with pytest.raises(GenerationError, match="decode_steps_per_launch"):
        scheduler(FakeRunner(script), decode_steps_per_launch=0)
    # a step function that also samples on the device is handed every request's temperature, seed and draws so far
    runner = SeveralStepsRunner(script)
    runner.decode_steps_sample = True
    s = scheduler(runner, decode_steps_per_launch=2)
    s.add_request([3, 4], max_new_tokens=4, sampling=SamplingConfig(temperature=0.7, seed=11))
    s.add_request([5], max_new_tokens=4)
    drain(s)
    assert runner.launches == [(2, [0, 1])]
    (first, second), = runner.sampling_seen
    assert first == (0.7, 11, 1) and second[0] == 0.0 and second[2] == 1


class QueuedLaunchRunner(SeveralStepsRunner):
    """A fake step function whose launches of decode steps can be queued and waited for later, as the real one's: a
    launch that follows another takes its first tokens from that one (the entries' own are not read), and only the
    launch begun last can be followed."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.begun, self.ended, self.dropped, self.serial, self.open = [], [], [], 0, 0
        self.decode_steps_sample = True

    def step(self, entries):
        assert self.open == 0, "a step ran while a launch was in flight"
        self.serial += 1
        return super().step(entries)

    def decode_launch_begin(self, entries, steps, sampling=None, after=None):
        if after is not None:
            assert after["serial"] == self.serial and [e.cache for e in entries] == [e.cache for e in after["entries"]]
        for e in entries:
            self.cache.extend(e.cache, steps)          # a released cache would refuse
        self.serial += 1
        self.open += 1
        launch = {"entries": list(entries), "steps": steps, "serial": self.serial, "follows": after is not None, "sampled": False}
        launch = type("Launch", (), launch)() if False else _Launch(launch)
        self.begun.append((steps, [e.cache.request_id for e in entries], after is not None))
        return launch

    def decode_launch_end(self, launch):
        self.open -= 1
        self.ended.append(launch.serial)
        chosen = []
        for _ in range(launch.steps):
            row = []
            for e in launch.entries:
                k = self.produced.get(e.cache.request_id, 0)
                self.produced[e.cache.request_id] = k + 1
                script = self.script[e.cache.request_id]
                row.append(script[k] if k < len(script) else 0)
            chosen.append(row)
        self.cache.check_invariants()
        return chosen

    def decode_launch_drop(self, launch):
        self.open -= 1
        self.dropped.append(launch.serial)


class _Launch(dict):
    __getattr__ = dict.__getitem__


def test_launches_queued_ahead_give_the_same_events_and_end_their_chain_when_a_request_ends():
    # request 1 meets its end-of-sequence token as its sixth token, inside the second launch
    script = {0: list(range(10, 40)), 1: [20, 21, 22, 23, 24, 1] + [9] * 30}

    def run(ahead):
        runner = QueuedLaunchRunner(script)
        s = scheduler(runner, decode_steps_per_launch=4, launch_ahead=ahead)
        s.add_request([3, 4, 5], max_new_tokens=18)
        s.add_request([6, 2], max_new_tokens=18)
        events = [(i, e.token_id, e.token_index, e.finish_reason) for i, e in drain(s)]
        assert runner.cache.active_requests == 0 and runner.cache.used_pages() == 0 and runner.open == 0
        return events, runner, s

    plain, _, log_plain = run(False)
    ahead, runner, log_ahead = run(True)
    assert sorted(plain) == sorted(ahead) and log_plain.step_log == log_ahead.step_log
    assert [t for i, t, _, _ in ahead if i == 1] == [20, 21, 22, 23, 24, 1]
    # Both requests have sampled once when the launches begin.  The first (tokens 2..5) is followed at once by a second
    # (6..9) and, when the first is read, a third (10..13) behind the second.  Request 1 ends in the second; the third,
    # already queued with it, is the last of its chain, and request 1's rows of it are dropped.  Request 0 (13 tokens
    # so far, 5 to go) goes on alone: a launch of 4 and, behind it, one of the single token that is left.
    assert runner.begun == [(4, [0, 1], False), (4, [0, 1], True), (4, [0, 1], True), (4, [0], False), (1, [0], True)]
    assert runner.dropped == [] and len(runner.ended) == 5
    assert [t for i, t, _, _ in ahead if i == 0] == list(range(10, 28))


def test_launches_are_not_queued_ahead_past_a_length_limit_or_while_a_request_could_be_admitted():
    script = {0: list(range(10, 40)), 1: list(range(40, 70)), 2: [7] * 10}
    runner = QueuedLaunchRunner(script, num_pages=40)
    s = scheduler(runner, decode_steps_per_launch=4, launch_ahead=True, max_batch_size=2)
    s.add_request([3, 4], max_new_tokens=7)            # six tokens after the first: a launch of 4, then 2 are left
    s.add_request([5, 6], max_new_tokens=30)
    s.add_request([8, 9], max_new_tokens=3)            # waits for a slot
    events = drain(s)
    # the launch of 4 is followed by one of 2 (what request 0 has left); when request 0 ends, the waiting request
    # could be admitted, so nothing is queued behind the launch in flight and the next step takes it in
    assert runner.begun[:2] == [(4, [0, 1], False), (2, [0, 1], True)]
    assert all(not follows for _, ids, follows in runner.begun[2:3])
    assert {i for i, _ in events} == {0, 1, 2} and runner.open == 0 and runner.cache.used_pages() == 0
    assert [e.token_id for i, e in events if i == 2] == [7, 7, 7]


def test_a_launch_in_flight_is_waited_for_when_everything_is_given_up():
    script = {0: list(range(10, 40)), 1: list(range(40, 70))}
    runner = QueuedLaunchRunner(script)
    s = scheduler(runner, decode_steps_per_launch=4, launch_ahead=True)
    s.add_request([3, 4], max_new_tokens=20)
    s.add_request([5, 6], max_new_tokens=20)
    while not runner.begun:
        s.step()
    assert runner.open == 1                              # one launch has been read, the one behind it is in flight
    s.abort_all()
    assert runner.open == 0 and len(runner.dropped) == 1 and runner.cache.used_pages() == 0 and not s.has_unfinished
