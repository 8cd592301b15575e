"""The step function: one batch of (request, its next tokens) through the model.

A step is a list of StepEntry(cache, tokens, want).  A prompt portion and a decoded token
are the same thing with different lengths; entries may be cut anywhere.  The runner

  1. extends every request's cache by its tokens (taking pages as needed),
  2. writes the step's metadata into one pinned host buffer and copies it to the device once,
  3. runs the model on exactly the step's tokens as one ragged batch, reading earlier
     positions from the paged cache,
  4. returns float32 logits at the wanted places, in entry order then `want` order,
  5. on failure rolls every cache back to its length before the step.

Device metadata (all int32): token ids, positions, request row of each token, the state slot of
each token's request (which is also its row in the block tables), rows whose logits are wanted,
per request cumulative query starts, context lengths and state slots, and per cache group the
physical slot of each token.  The block tables themselves stay on the device (cache/manager.py):
the step sends the entries that changed since the last one behind its metadata, in the same copy,
and a small kernel writes them in before the step's own kernels run.  The layout has fixed offsets
given the capacities, so a captured graph can be replayed after only the buffer's content has changed.

Reference: mini_llm/model/base.py:161-248 (prefill/decode as extend -> forward -> logits,
rollback on failure); the reference runs whole prompts alone and decode tokens as a second
kind of call, here both are one call.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import ctypes

import numpy as np
import torch

from ..cache import CacheManager, RequestCache
from ..errors import GenerationError, KVCacheError
from ..kernels import ops
from ..models import DecoderModel
from ..parts.base import length_class
from ..sampling.sampler import refuse_not_finite


@dataclass
class StepEntry:
    cache: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = ()


class GroupStep:
    """Per cache group view of the step metadata on the device: the cache slot of every token of the step, and the
    group's block table [max_requests + 1, max_blocks], whose row for a token is ctx.token_slot[token]."""

    def __init__(self, slots: torch.Tensor, block_table: torch.Tensor, page_size: int):
        self.slots, self.block_table, self.page_size = slots, block_table, page_size


class ScratchArena:
    """Named device buffers that live across steps, so that a step allocates nothing once warm."""

    def __init__(self, device):
        self.device = device
        self._buffers: dict = {}
        # bumped whenever a buffer that was handed out before is replaced by a larger one: whoever wrote its
        # address down (a captured graph, a recorded plan) then holds a stale address.  A buffer made for
        # the first time moves nothing.
        self.generation = 0

    def get(self, name: str, shape: tuple, dtype: torch.dtype, zeroed: bool = False) -> torch.Tensor:
        """The buffer `name` with at least shape[0] rows.  zeroed: all zero when it is made (for buffers whose
        users leave them as they found them, such as arrival counters); never cleared again."""
        rows, rest = shape[0], tuple(shape[1:])
        key = (name, rest, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.shape[0] < rows:
            capacity = max(rows, 1 if buf is None else buf.shape[0] * 2)
            if buf is not None:
                self.generation += 1
            buf = (torch.zeros if zeroed else torch.empty)((capacity, *rest), dtype=dtype, device=self.device)
            self._buffers[key] = buf
        return buf[:rows]

    def reserve(self, name: str, shape: tuple, dtype: torch.dtype) -> None:
        self.get(name, shape, dtype)

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._buffers.values())


@dataclass
class RecordedStep:
    """The launches of one step shape, written down (see ModelRunner._step_eager)."""

    plan: "ops.Plan"
    generation: int                      # of the scratch arena when it was recorded
    logits: torch.Tensor | None          # where the step's logits come out
    uses: int = 0
    graph: int | None = None             # the plan captured in a HIP graph, once the shape has come back often enough


@dataclass
class DecodeLaunch:
    """Decode steps that have been queued and not yet waited for (ModelRunner.decode_launch_begin)."""

    entries: list
    steps: int
    bucket: int
    before: list                         # the caches' lengths before the launch
    ctx: "StepContext"
    sampled: bool
    parity: int                          # which of the two result buffers its tokens go to
    done: object                         # an event recorded behind the launch
    serial: int
    ended: bool = False


class StepContext:
    """What the parts see of one step."""

    def __init__(self, runner: "ModelRunner"):
        self._runner = runner
        self.kernels = runner.kernels          # which matrix-product kernels this runner's steps use (ops.KernelChoice)
        self.dtype = runner.dtype
        self.device = runner.device
        self.memo: dict = {}
        self.T = self.R = self.num_logit_rows = self.num_qblocks = self.max_qblock = 0
        self.qblock_token0 = self.qblock_count = None
        self.max_q = self.max_k = self.max_k_bound = 0
        self.all_decode = False
        self.single_rows = 0          # a mixed step's leading requests that bring one token each (their tokens are its first rows)
        self.host_q_lens: list[int] = []
        self.host_slots: list[int] = []
        self.host_positions: list[int] = []   # first position of each request's tokens in this step
        self.token_ids = self.positions = self.token_request = self.token_slot = self.logit_rows = None
        self.cu_seqlens_q = self.seq_lens_k = self.slot_ids = self.counts = None
        self._groups: list[GroupStep] = []

    def scratch(self, name: str, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        return self._runner.arena.get(name, shape, dtype)

    def group(self, index: int) -> GroupStep:
        return self._groups[index]

    def layer_cache(self, schedule_position: int):
        return self._runner.cache.layer_caches[schedule_position]


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, *, max_step_tokens: int, dtype: torch.dtype, device,
                 use_graph: bool = False, library_gemm: bool = True, kernels: "ops.KernelChoice | None" = None,
                 use_plans: bool = True):
        if max_step_tokens <= 0:
            raise GenerationError(f"max_step_tokens must be positive, got {max_step_tokens}")
        self.model, self.cache, self.dtype, self.device = model, cache, dtype, torch.device(device)
        self.max_step_tokens = max_step_tokens
        self.max_requests = cache.max_requests
        self.arena = ScratchArena(self.device)
        # Which matrix-product kernels this runner's steps use: a property of the runner, carried by every step's
        # context, never of the process.  Unless `kernels` says otherwise: bfloat16 products of more rows than this
        # package's kernels for few rows take go to the vendor library, if `library_gemm` allows it.
        self._graphs: dict[tuple, tuple] = {}   # (bucket, length class) -> (handle, arena generation, logits tensor)
        self._plans: dict[tuple, RecordedStep] = {}
        self._kernels = kernels if kernels is not None else ops.KernelChoice(library=library_gemm)
        self.library_gemm = self.kernels.library
        # decode-only steps are captured in a HIP graph per padded batch size and replayed
        self.use_graph = use_graph and model.graph_safe()
        # Steps that are not replayed from a graph (prompt portions, mixed steps) are recorded as launch plans:
        # the first step of a shape runs through the parts as usual while every launch is written down; later
        # steps of that shape fill in the metadata and make the same launches from one call into the library.
        # A shape is what the launches' arguments depend on (see _plan_key); a plan also names addresses, so it
        # is good only while the scratch buffers stay where they are (the arena's generation).  Only models
        # whose every part launches through this package's kernels alone (`plan_safe`) are recorded.
        self._use_plans = use_plans and getattr(model, "plan_safe", lambda: False)()
        self.plan_replays = 0
        self.plan_recordings = 0
        self.plan_graph_replays = 0     # of the replays, those made by launching the graph of a plan
        self.graph_replays = 0     # steps (or launches of several steps) served by replaying a graph
        self.graph_captures = 0    # ... and those that ran eagerly and were captured on the way
        # query groups for mixers that ask for them (the ragged attention kernel): at most `query_group` consecutive
        # tokens of one request
        self._query_groups = getattr(model, "wants_query_groups", lambda: True)()
        self.query_group = ops.attention_prefill_group() if self._query_groups else 0   # the most; a step of few tokens uses smaller ones
        # The metadata of a step is one int32 buffer whose layout follows the step's own numbers of
        # tokens and requests, so that a decode step uploads a few KB whatever the limits are.  A
        # graph holds addresses inside it: steps of one padded batch size share one layout.
        self._layouts: dict[tuple[int, int], tuple[dict, int]] = {}
        self._off, self._meta_size = self._layout(max_step_tokens, self.max_requests)
        # behind a step's arrays: the block table entries that changed since the last step, as (offset, value) pairs
        cursor = self._meta_size + 2 * self.TABLE_PATCHES + 4
        self._patches = 0
        # two pinned staging buffers used in turn: a buffer is rewritten only after the copy
        # that read it has finished
        pin = self.device.type == "cuda"
        self._hosts = [torch.zeros(cursor, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        if pin and not all(host.is_pinned() for host in self._hosts):
            raise GenerationError("could not allocate pinned host memory for the step metadata")
        self._copied = [None, None]
        self._turn = 0
        self._host = self._hosts[0]
        self._host_np = self._host.numpy()
        self._dev = torch.zeros(cursor, dtype=torch.int32, device=self.device)
        self._views: dict[tuple, tuple] = {}
        self._chosen_devs = self._chosen_hosts = None   # tokens chosen on the device by decode_steps(): two sets, for launches that follow each other
        self._launch_serial = 0     # counts everything that writes the device's step metadata
        self._sampling_dev = self._sampling_host = None
        self._counting = np.arange(max(max_step_tokens, self.max_requests) + 1, dtype=np.int32)
        # the staging buffer is filled by the library's host routine; False: by the Python routine it is tested against
        self.native_prepare = True
        self._native_layouts: dict = {}
        self._summary = np.zeros(ops.step_prepare_summary_size(), dtype=np.int32)
        self._table_addresses = (ctypes.c_void_p * max(len(cache.groups), 1))(*[cache.tables_with_trash_row(i).ctypes.data for i in range(len(cache.groups))])
        self.steps_run = 0
        # The weights, the cache pools and the buffers above were converted and cleared by work queued
        # on the stream that is current now.  A step on another stream waits for that work once: streams
        # made by torch do not wait for the default stream by themselves.
        self._built = None
        if self.device.type == "cuda":
            stream = torch.cuda.current_stream(self.device)
            self._built = torch.cuda.Event()
            self._built.record(stream)
            self._follows_construction = {stream.cuda_stream}

    # A captured graph and a recorded plan hold the kernels that were chosen when they were made, and the addresses of
    # the weights and pages of that time: whoever changes the choice gets them made again.
    @property
    def kernels(self) -> "ops.KernelChoice":
        return self._kernels

    @kernels.setter
    def kernels(self, choice: "ops.KernelChoice") -> None:
        if choice != self._kernels:
            self.drop_graphs()
        self._kernels = choice
        self.library_gemm = choice.library

    @property
    def use_plans(self) -> bool:
        return self._use_plans

    @use_plans.setter
    def use_plans(self, wanted: bool) -> None:
        wanted = bool(wanted) and getattr(self.model, "plan_safe", lambda: False)()
        if wanted != self._use_plans:
            self.drop_graphs()
        self._use_plans = wanted

    def _layout(self, tokens: int, requests: int) -> tuple[dict, int]:
        """Where each array of a step of `tokens` tokens and `requests` requests lies in the metadata
        buffer: name -> (first element, elements), and the elements in all (16-byte aligned parts)."""
        known = self._layouts.get((tokens, requests))
        if known is None:
            offsets, cursor = {}, 0
            qblocks = -(-tokens // 16) + requests if self._query_groups else 0
            parts = [("token_ids", tokens), ("positions", tokens), ("token_request", tokens), ("token_slot", tokens), ("logit_rows", tokens),
                     ("cu_seqlens_q", requests + 1), ("seq_lens_k", requests), ("slot_ids", requests),
                     ("qblock_token0", qblocks), ("qblock_count", qblocks), ("counts", 4)]
            for index in range(len(self.cache.groups)):
                parts += [(f"slots{index}", tokens)]
            for name, size in parts:
                offsets[name] = (cursor, size)
                cursor += -(-size // 4) * 4
            known = self._layouts[(tokens, requests)] = (offsets, cursor)
        return known

    def _follow_construction(self) -> None:
        """Order the current stream after the work that built the model, the cache and this runner."""
        if self._built is None:
            return
        if self._built.query():
            self._built = None
            return
        stream = torch.cuda.current_stream(self.device)
        if stream.cuda_stream not in self._follows_construction:
            stream.wait_event(self._built)
            self._follows_construction.add(stream.cuda_stream)

    def _next_staging(self) -> None:
        self._turn ^= 1
        if self._copied[self._turn] is not None:
            self._copied[self._turn].synchronize()
        self._host = self._hosts[self._turn]
        self._host_np = self._host.numpy()

    TABLE_PATCHES = 2048     # block table entries a step's metadata has room for (more are sent as the whole tables, once)

    def _stage_table_patches(self) -> None:
        """The block table entries that changed on the host since the last step, behind the step's arrays."""
        self._patches = 0
        changed = self.cache.table_patches() if self.cache.device_tables is not None else None
        if changed is None:
            return
        offsets, values = changed
        if len(offsets) > self.TABLE_PATCHES:
            self.cache.upload_tables()
            return
        pairs = self._host_np[self._meta_size:self._meta_size + 2 * len(offsets)]
        pairs[0::2], pairs[1::2] = offsets, values
        self._patches = len(offsets)

    def _upload(self) -> None:
        self._stage_table_patches()
        if self._patches and self._meta_size <= 65536:
            # the same launch writes the changed block table entries, which it reads where the host put them
            ops.copy_h2d_scatter(self._dev, self._host, self._meta_size, self.cache.device_tables, self._meta_size, self._patches)
        elif self._patches:   # a step of tens of thousands of tokens: the runtime's copy, the pairs with it, then the scatter
            ops.copy_h2d(self._dev, self._host, -(-(self._meta_size + 2 * self._patches) // 4) * 4)
            ops.scatter_i32(self.cache.device_tables, self._dev, self._patches, first=self._meta_size)
        else:
            ops.copy_h2d(self._dev, self._host, self._meta_size)
        self._launch_serial += 1          # the device's step metadata is another step's now
        self._mark_copied()

    def _mark_copied(self) -> None:
        if self.device.type == "cuda":
            event = self._copied[self._turn] or torch.cuda.Event()
            event.record()
            self._copied[self._turn] = event

    def _view(self, name: str, count: int | None = None) -> torch.Tensor:
        start, size = self._off[name]
        return self._dev[start:start + (size if count is None else count)]

    def _host_view(self, name: str) -> np.ndarray:
        start, size = self._off[name]
        return self._host_np[start:start + size]

    # -------------------------------------------------------------------- step
    def validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise GenerationError("a step needs at least one entry")
        if len(entries) > self.max_requests:
            raise GenerationError(f"a step holds {len(entries)} requests but at most {self.max_requests} fit")
        total = 0
        seen = set()
        vocab = self.model.spec.vocab_size
        for entry in entries:
            n = len(entry.tokens)
            if n == 0:
                raise GenerationError("every entry of a step needs at least one token")
            if id(entry.cache) in seen:
                raise GenerationError("a request may appear only once in a step")
            seen.add(id(entry.cache))
            if min(entry.tokens) < 0 or max(entry.tokens) >= vocab:
                raise GenerationError(f"input_ids must be within vocabulary [0, {vocab})")
            for place in entry.want:
                if not 0 <= place < n:
                    raise GenerationError(f"wanted place {place} is outside the entry's {n} tokens")
            total += n
        if total > self.max_step_tokens:
            raise GenerationError(f"a step holds {total} tokens but at most {self.max_step_tokens} fit")

    def prepare(self, entries: Sequence[StepEntry], pad_to: int = 0, ahead: int = 0) -> StepContext:
        """Fill the host metadata for `entries` (caches already extended) and copy it over.

        With `pad_to` (decode-only steps) the batch is filled up to that many rows with rows that
        belong to no request: token 0 at position 0, written to and read from the trash page, and
        logits are produced for every row, so that the step's shape depends on `pad_to` alone.
        `ahead` (decode-only steps): the caches were extended by that many positions more than this
        step's one, for the steps that follow it in the same launch; positions and context lengths are
        this step's, the block tables hold the later pages too."""
        cache, page = self.cache, self.cache.page_size
        ctx = StepContext(self)
        self._next_staging()
        self._off, self._meta_size = self._layout(max(sum(len(e.tokens) for e in entries), pad_to), max(len(entries), pad_to))
        if self.native_prepare:
            self._prepare_native(ctx, entries, pad_to, ahead)
        else:
            self._prepare_python(ctx, entries, pad_to, ahead)
        # what kernels size their tables and choose their key splits by: an upper bound of the longest context that is
        # the same for every step of one shape (a recorded plan holds it), the next multiple of 256
        ctx.max_k_bound = min(-(-ctx.max_k // 256) * 256, max(cache.max_seq_len, ctx.max_k))
        if pad_to:
            # a graph outlives the step it is captured in: sizes that must hold for every replay are
            # made for the longest context the cache can hold
            ctx.max_k_bound = cache.max_seq_len
        ctx.all_decode = ctx.max_q == 1
        self._upload()
        self.bind_views(ctx)
        return ctx

    def _prepare_native(self, ctx: StepContext, entries: Sequence[StepEntry], pad_to: int, ahead: int) -> None:
        """The staging buffer filled by the library's host routine (csrc/prepare.hip) from the entries as flat arrays."""
        count = len(entries)
        ctx.host_slots = [entry.cache.slot for entry in entries]
        lengths = [entry.cache.length - ahead for entry in entries]
        ctx.host_q_lens = [len(entry.tokens) for entry in entries]
        wants = [len(entry.want) for entry in entries]
        if ahead and any(n != 1 for n in ctx.host_q_lens):
            raise GenerationError("only a decode-only step can be prepared ahead of later steps")
        flat = ctx.host_slots + lengths + ctx.host_q_lens + wants
        for entry in entries:
            flat += entry.tokens
        for entry in entries:
            flat += entry.want
        packed = np.array(flat, dtype=np.int32)
        tokens_at = 4 * count
        wants_at = tokens_at + sum(ctx.host_q_lens)
        offsets, tables = self._native_layout()
        summary = self._summary
        ops.step_prepare(self._host_np, offsets, count, packed, tokens_at, wants_at, pad_to, self.cache.trash_slot, tables,
                         len(self.cache.groups), self.cache.max_blocks, self.cache.page_size, self.query_group if self._query_groups else 0, summary)
        (ctx.T, ctx.R, ctx.num_logit_rows, ctx.num_qblocks, ctx.max_qblock, ctx.max_q, ctx.max_k, ctx.single_rows) = summary.tolist()
        ctx.host_positions = [length - n for length, n in zip(lengths, ctx.host_q_lens)]

    def _native_layout(self):
        """The current layout's offsets in the order the host routine reads them, and the host block tables' addresses."""
        known = self._native_layouts.get(id(self._off))
        if known is None:
            names = ["token_ids", "positions", "token_request", "token_slot", "logit_rows", "cu_seqlens_q", "seq_lens_k", "slot_ids",
                     "qblock_token0", "qblock_count", "counts"] + [f"slots{i}" for i in range(len(self.cache.groups))]
            known = self._native_layouts[id(self._off)] = np.array([self._off[name][0] for name in names], dtype=np.int64)
        return known, self._table_addresses

    def _prepare_python(self, ctx: StepContext, entries: Sequence[StepEntry], pad_to: int, ahead: int) -> None:
        """The same in Python and numpy: the reference the host routine is tested against."""
        cache, page = self.cache, self.cache.page_size
        ids, pos, req, rows = (self._host_view(n) for n in ("token_ids", "positions", "token_request", "logit_rows"))
        cu, lens, slots, of_token = (self._host_view(n) for n in ("cu_seqlens_q", "seq_lens_k", "slot_ids", "token_slot"))
        cursor = n_rows = 0
        cu[0] = 0
        if all(len(entry.tokens) == 1 for entry in entries):
            # one token per request (a decode step): whole arrays at once, no loop over tokens
            cursor = len(entries)
            count = self._counting[:cursor + 1]
            lengths = np.fromiter((entry.cache.length - ahead for entry in entries), dtype=np.int32, count=cursor)
            ctx.host_slots = [entry.cache.slot for entry in entries]
            ids[:cursor] = [entry.tokens[0] for entry in entries]
            pos[:cursor] = lengths - 1
            req[:cursor] = count[:cursor]
            cu[:cursor + 1] = count
            lens[:cursor] = lengths
            slots[:cursor] = ctx.host_slots
            of_token[:cursor] = ctx.host_slots
            wanted = [r for r, entry in enumerate(entries) for _ in entry.want]   # a place asked twice is given twice
            n_rows = len(wanted)
            rows[:n_rows] = wanted
            ctx.host_q_lens = [1] * cursor
            ctx.host_positions = pos[:cursor].tolist()
        else:
            if ahead:
                raise GenerationError("only a decode-only step can be prepared ahead of later steps")
            for r, entry in enumerate(entries):
                n = len(entry.tokens)
                start = entry.cache.length - n
                ids[cursor:cursor + n] = entry.tokens
                pos[cursor:cursor + n] = np.arange(start, start + n, dtype=np.int32)
                req[cursor:cursor + n] = r
                of_token[cursor:cursor + n] = entry.cache.slot
                for place in entry.want:
                    rows[n_rows] = cursor + place
                    n_rows += 1
                cu[r + 1] = cursor + n
                lens[r] = entry.cache.length
                slots[r] = entry.cache.slot
                ctx.host_q_lens.append(n)
                ctx.host_slots.append(entry.cache.slot)
                ctx.host_positions.append(start)
                cursor += n
        real = len(entries)
        ctx.max_q = max(ctx.host_q_lens)
        ctx.max_k = int(lens[:real].max())
        ctx.all_decode = ctx.max_q == 1
        if pad_to > real:
            extra = pad_to - real
            ids[cursor:cursor + extra] = 0
            pos[cursor:cursor + extra] = 0
            req[cursor:cursor + extra] = np.arange(real, pad_to, dtype=np.int32)
            cu[real + 1:pad_to + 1] = np.arange(cursor + 1, cursor + extra + 1, dtype=np.int32)
            lens[real:pad_to] = 1
            slots[real:pad_to] = cache.trash_slot        # their state, like their keys and values, goes where no request reads
            of_token[cursor:cursor + extra] = cache.trash_slot   # ... and the trash row of the block tables names the trash page
            cursor += extra
        if pad_to:
            rows[:cursor] = np.arange(cursor, dtype=np.int32)
            n_rows = cursor
        ctx.T, ctx.R, ctx.num_logit_rows = cursor, max(real, pad_to), n_rows
        self._host_view("counts")[0] = real          # rows that belong to requests (the others pad a graph's batch)
        # groups of consecutive tokens of one request, the longest contexts first: only for mixers that ask for them
        if not self._query_groups:
            ctx.num_qblocks = ctx.max_qblock = 0
        elif ctx.all_decode:
            ctx.num_qblocks, ctx.max_qblock = cursor, 1
            self._host_view("qblock_token0")[:cursor] = np.argsort(-pos[:cursor], kind="stable")
            self._host_view("qblock_count")[:cursor] = 1
        else:
            # The requests at the head of the step that bring one token each (a scheduler puts its decoding requests
            # first) are left to the mixer as single rows, `single_rows` of them: the query groups cover the rows
            # after them, and count their tokens from there.
            singles = next(i for i, n in enumerate(ctx.host_q_lens) if n != 1)
            ctx.single_rows = singles
            starts, size = cu[:ctx.R + 1], min(self.query_group, ops.attention_prefill_group(cursor - singles, ctx.max_k))
            blocks = [(int(pos[min(t0 + size, int(starts[i + 1])) - 1]), t0 - singles, min(size, int(starts[i + 1]) - t0))
                      for i in range(singles, ctx.R) for t0 in range(int(starts[i]), int(starts[i + 1]), size)]
            blocks.sort(key=lambda b: -b[0])
            ctx.num_qblocks = len(blocks)
            ctx.max_qblock = max(b[2] for b in blocks)
            self._host_view("qblock_token0")[:len(blocks)] = [b[1] for b in blocks]
            self._host_view("qblock_count")[:len(blocks)] = [b[2] for b in blocks]
        for index, group in enumerate(cache.groups):
            gslots = self._host_view(f"slots{index}")
            p = pos[:cursor]
            pages = cache.tables_with_trash_row(index)[of_token[:cursor], p // page]
            gslots[:cursor] = np.where(pages >= 0, pages * page + p % page, -1)

    def bind_views(self, ctx: StepContext) -> None:
        """The device views of the step's arrays; steps of one shape share them (slicing is slow)."""
        key = (ctx.T, ctx.R, ctx.num_logit_rows, ctx.num_qblocks)
        views = self._views.get(key)
        if views is None:
            if len(self._views) > 256:
                self._views.clear()
            views = self._views[key] = (
                self._view("token_ids", ctx.T), self._view("positions", ctx.T), self._view("token_request", ctx.T), self._view("token_slot", ctx.T),
                self._view("logit_rows", max(ctx.num_logit_rows, 1)), self._view("cu_seqlens_q", ctx.R + 1),
                self._view("seq_lens_k", ctx.R), self._view("slot_ids", ctx.R), self._view("qblock_token0", ctx.num_qblocks),
                self._view("qblock_count", ctx.num_qblocks), self._view("counts", 4),
                [GroupStep(self._view(f"slots{i}", ctx.T), self.cache.device_table(i), self.cache.page_size)
                 for i in range(len(self.cache.groups))])
        (ctx.token_ids, ctx.positions, ctx.token_request, ctx.token_slot, ctx.logit_rows, ctx.cu_seqlens_q, ctx.seq_lens_k, ctx.slot_ids,
         ctx.qblock_token0, ctx.qblock_count, ctx.counts, ctx._groups) = views

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        """Run one step; returns float32 logits [wanted, vocab] on the device, or None if none is wanted.

        The logits lie in a buffer that the next step writes again: read or copy them before it."""
        self.validate(entries)
        self._follow_construction()
        before = [entry.cache.length for entry in entries]
        extended = []
        states = self.cache.snapshot_state([entry.cache for entry in entries])
        try:
            for entry in entries:
                self.cache.extend(entry.cache, len(entry.tokens))
                extended.append(entry)
            bucket = self._graph_bucket(entries)
            if bucket:
                logits = self._step_graph(entries, bucket)
            else:
                logits = self._step_eager(self.prepare(entries))
        except BaseException:       # an interrupt from the keyboard in the middle of a step must leave no trace either
            ops.record_drop()
            self._undo(extended, before, states)
            raise
        for entry in entries:
            self.cache.trim(entry.cache)
        self.steps_run += 1
        return logits

    def _plan_key(self, ctx: StepContext) -> tuple:
        """Everything the launches of a step depend on besides the contents of the metadata buffer: the numbers
        of tokens, requests, wanted rows and query groups (sizes and grids, and where the metadata arrays lie),
        the largest query group, whether every request brings one token, how many at the head of a mixed step do,
        and the two coarse measures of the longest context that kernels size tables and choose key splits by."""
        return (ctx.T, ctx.R, ctx.num_logit_rows, ctx.num_qblocks, ctx.max_qblock, ctx.all_decode, ctx.single_rows, ctx.max_k_bound,
                length_class(ctx.max_k))

    def _step_eager(self, ctx: StepContext) -> torch.Tensor | None:
        """The model on a prepared step, outside any graph: from a recorded plan if one fits, else through
        the parts (recording a plan on the way, if plans are in use)."""
        if not self.use_plans:
            h = self.model.forward_hidden(ctx)
            return self.model.logits(ctx, h) if ctx.num_logit_rows else None
        key = self._plan_key(ctx)
        known = self._plans.get(key)
        if known is not None and known.generation == self.arena.generation:
            known.uses += 1
            stream = torch.cuda.current_stream(self.device).cuda_stream
            if known.graph is None and known.uses >= self.PLAN_GRAPH_AFTER and stream != 0:
                # a shape that keeps coming back: its launches go into a HIP graph, made by running the plan under
                # capture (nothing runs then), and from now on the step is one graph launch
                ops.graph_begin()
                try:
                    ops.plan_run(known.plan)
                except BaseException:
                    ops.graph_destroy(ops.graph_end())
                    raise
                known.graph = ops.graph_end()
            if known.graph is not None and stream != 0:
                ops.graph_launch(known.graph)
                self.plan_graph_replays += 1
            else:
                ops.plan_run(known.plan)
            self.plan_replays += 1
            return known.logits
        if known is not None:
            self._forget_plan(key)
        generation = self.arena.generation
        ops.record_begin()
        try:
            h = self.model.forward_hidden(ctx)
            logits = self.model.logits(ctx, h) if ctx.num_logit_rows else None
        except BaseException:
            ops.record_drop()
            raise
        plan = ops.record_end()
        if self.arena.generation == generation:          # else a buffer moved on the way: addresses written down before are stale
            if len(self._plans) >= self.MAX_PLANS:
                self._forget_plan(next(iter(self._plans)))
            self._plans[key] = RecordedStep(plan, generation, logits)
            self.plan_recordings += 1
        return logits

    def _forget_plan(self, key: tuple) -> None:
        known = self._plans.pop(key, None)
        if known is not None and known.graph is not None:
            if self.device.type == "cuda":
                torch.cuda.synchronize(self.device)
            ops.graph_destroy(known.graph)

    PLAN_GRAPH_AFTER = 3     # replays of a plan after which it is captured in a graph
    MAX_PLANS = 512      # plans kept (each a few hundred launches of a few dozen words); the oldest goes first

    def _undo(self, extended: Sequence[StepEntry], before: Sequence[int], states: list) -> None:
        """After a failed step: every cache that was extended back to its length before the step (pages
        that only the step took go back to the pool) and every per-request state row as it was."""
        for entry, length in zip(extended, before):
            if not entry.cache.released:
                self.cache.rollback(entry.cache, length)
        self.cache.restore_state(states)

    # ------------------------------------------------- several decode steps, one launch
    MAX_DECODE_STEPS = 8
    GRAPH_ROWS = 128    # largest padded batch whose bfloat16 step is captured

    def can_decode_steps(self, entries: Sequence[StepEntry]) -> bool:
        """Whether decode_steps() takes these entries: one token each, and a graph for their number."""
        return self._graph_bucket(entries) > 0

    decode_steps_sample = True     # decode_steps() also draws from filtered, tempered distributions

    def decode_steps(self, entries: Sequence[StepEntry], steps: int, sampling: Sequence | None = None) -> list[list[int]]:
        """`steps` decode steps of the same requests, the host out of the loop between them.

        Each entry brings the one token its request decodes next.  After every step the device itself
        chooses a token for every row (the largest logit; or, for the rows whose entry of `sampling`,
        a list of sampling.SamplingRow, says so, a seeded draw after top-k / top-p filtering, exactly
        as Sampler.choose would), feeds it in as the next token and moves the step's metadata one
        position on.  Returns the chosen tokens [steps][entries]; every request's cache is `steps`
        tokens longer afterwards, or, after a failure, as long as before.

        The steps run from one graph launch, unless the longest context crosses into another length
        class on the way (256, 512, 1024, ...): how far decode attention divides the keys follows the
        class, so the launch ends at the edge and another begins there.  Every step thus runs exactly
        as it would alone, and the tokens do not depend on how many steps a launch holds."""
        if not 1 <= steps <= self.MAX_DECODE_STEPS:
            raise GenerationError(f"decode_steps takes 1..{self.MAX_DECODE_STEPS} steps, got {steps}")
        self.validate(entries)
        self._follow_construction()
        bucket = self._graph_bucket(entries)
        if not bucket:
            raise GenerationError("decode_steps needs graphs and one token per entry")
        if sampling is not None and len(sampling) != len(entries):
            raise GenerationError("decode_steps needs one sampling row per entry")
        before = [entry.cache.length for entry in entries]
        states = self.cache.snapshot_state([entry.cache for entry in entries])
        chosen: list[list[int]] = []
        current, rows = list(entries), sampling
        try:
            while len(chosen) < steps:
                longest = max(entry.cache.length for entry in entries) + 1     # the longest context of the launch's first step
                reach = length_class(longest)
                edge = 2 * reach if reach else 256
                count = min(steps - len(chosen), edge - longest)
                if chosen:
                    current = [StepEntry(entry.cache, [token], entry.want) for entry, token in zip(entries, chosen[-1])]
                    if sampling is not None:
                        rows = [type(row)(row.config, row.seed, row.counter + len(chosen)) for row in sampling]
                chosen += self._decode_launch(current, count, rows, bucket)
        except BaseException:
            self._undo(entries, before, states)
            raise
        for entry in entries:
            self.cache.trim(entry.cache)
        self.steps_run += steps
        return chosen

    # ------------------------------------------ launches that follow each other without the host between them
    def decode_launch_begin(self, entries: Sequence[StepEntry], steps: int, sampling: Sequence | None = None,
                            after: "DecodeLaunch | None" = None) -> "DecodeLaunch":
        """Queue up to `steps` decode steps of `entries` (as decode_steps() would run them) and return at once;
        decode_launch_end() waits for them and gives their tokens.

        after: the launch that was begun last, with the same requests in the same order and not yet ended: this one
        then follows it directly.  Its first tokens are the ones the device chose last (the entries' own tokens are
        not read), and the host sends nothing but the block table entries of the new pages, so the device goes from
        one launch to the next without waiting for the host.  A launch ends at the edge of a length class like those
        of decode_steps(): `launch.steps` says how many steps it holds."""
        if not 1 <= steps <= self.MAX_DECODE_STEPS:
            raise GenerationError(f"a launch takes 1..{self.MAX_DECODE_STEPS} decode steps, got {steps}")
        if after is None:
            self.validate(entries)
        elif after.serial != self._launch_serial or len(entries) != len(after.entries) or any(
                mine.cache is not theirs.cache for mine, theirs in zip(entries, after.entries)):
            raise GenerationError("a launch can only follow the launch begun last (no other step since), with the same requests in the same order")
        self._follow_construction()
        bucket = self._graph_bucket(entries)
        if not bucket:
            raise GenerationError("decode launches need graphs and one token per entry")
        if sampling is not None and len(sampling) != len(entries):
            raise GenerationError("decode launches need one sampling row per entry")
        longest = max(entry.cache.length for entry in entries) + 1         # the longest context of the launch's first step
        reach = length_class(longest)
        count = min(steps, (2 * reach if reach else 256) - longest)
        before = [entry.cache.length for entry in entries]
        extended = []
        try:
            for entry in entries:
                self.cache.extend(entry.cache, count)
                extended.append(entry)
            sampled = sampling is not None and any(not row.config.greedy for row in sampling)
            if after is None:
                ctx = self.prepare(entries, pad_to=bucket, ahead=count - 1)
                if sampled:
                    self._upload_sampling(sampling)
                parity = 0
            else:
                # the device holds the step's metadata, moved on by the launch before; only new pages are news to it
                if sampled != after.sampled:
                    raise GenerationError("a launch that follows another samples as that one does")
                ctx, parity = after.ctx, after.parity ^ 1
                ctx.max_k = longest
                self._next_staging()
                self._stage_table_patches()
                if self._patches:
                    ops.copy_h2d_scatter(self._dev, self._host, 0, self.cache.device_tables, self._meta_size, self._patches)
                    self._mark_copied()
            self._launch_decode_graph(ctx, bucket, count, sampled, parity, goes_on=True, follows=after is not None)
        except BaseException:
            for entry, length in zip(extended, before):
                if not entry.cache.released:
                    self.cache.rollback(entry.cache, length)
            raise
        self._launch_serial += 1
        done = torch.cuda.Event()
        done.record()
        return DecodeLaunch(list(entries), count, bucket, before, ctx, sampled, parity, done, self._launch_serial)

    def decode_launch_end(self, launch: "DecodeLaunch") -> list[list[int]]:
        """Wait for a launch and return its tokens [steps][entries] (a row whose logits were not finite raises)."""
        if launch.ended:
            raise GenerationError("this launch has been ended before")
        launch.ended = True
        launch.done.synchronize()
        chosen = self._read_chosen(launch.bucket, launch.steps, len(launch.entries), launch.parity)
        for entry in launch.entries:
            if not entry.cache.released:
                self.cache.trim(entry.cache)
        self.steps_run += launch.steps
        return [row[:len(launch.entries)] for row in chosen]

    def decode_launch_drop(self, launch: "DecodeLaunch") -> None:
        """Wait for a launch whose tokens nobody wants any more (its requests are being given up)."""
        if not launch.ended:
            launch.ended = True
            launch.done.synchronize()

    def _decode_launch(self, entries: Sequence[StepEntry], steps: int, sampling: Sequence | None, bucket: int) -> list[list[int]]:
        """One graph launch of `steps` decode steps.  Every cache is lengthened by all `steps` positions
        first, so the block tables that the launch uploads already hold the pages of the later ones."""
        for entry in entries:
            self.cache.extend(entry.cache, steps)
        ctx = self.prepare(entries, pad_to=bucket, ahead=steps - 1)
        sampled = sampling is not None and any(not row.config.greedy for row in sampling)
        if sampled:
            self._upload_sampling(sampling)
        return [row[:len(entries)] for row in self._run_decode_graph(ctx, bucket, steps, sampled, len(entries))]

    def _upload_sampling(self, sampling: Sequence) -> None:
        """Temperature, top-p, top-k, draws so far and seed of every row, in one buffer on the device
        (rows beyond those given stay at temperature 0: the largest logit)."""
        cap = -(-self.max_requests // 4) * 4
        if self._sampling_host is None:
            self._sampling_host = torch.zeros(6 * cap, dtype=torch.int32, pin_memory=True)
            self._sampling_dev = torch.zeros(6 * cap, dtype=torch.int32, device=self.device)
        host = self._sampling_host.numpy()
        host[:] = 0
        n = len(sampling)
        host[:cap].view(np.float32)[:n] = [row.config.temperature for row in sampling]
        host[cap:2 * cap].view(np.float32)[:n] = [row.config.top_p for row in sampling]
        host[2 * cap:3 * cap][:n] = [row.config.top_k or 0 for row in sampling]
        host[3 * cap:4 * cap][:n] = [row.counter for row in sampling]
        host[4 * cap:6 * cap].view(np.int64)[:n] = [row.seed for row in sampling]
        ops.copy_h2d(self._sampling_dev, self._sampling_host, 6 * cap)

    def _sampling_views(self, rows: int):
        cap = -(-self.max_requests // 4) * 4
        dev = self._sampling_dev
        return (dev[:cap].view(torch.float32)[:rows], dev[cap:2 * cap].view(torch.float32)[:rows], dev[2 * cap:3 * cap][:rows],
                dev[3 * cap:4 * cap][:rows], dev[4 * cap:6 * cap].view(torch.int64)[:rows])

    def _run_decode_graph(self, ctx: StepContext, bucket: int, steps: int, sampled: bool = False, real: int | None = None) -> list[list[int]]:
        self._launch_decode_graph(ctx, bucket, steps, sampled)
        torch.cuda.current_stream(self.device).synchronize()
        return self._read_chosen(bucket, steps, bucket if real is None else real)

    def _read_chosen(self, bucket: int, steps: int, real: int, parity: int = 0) -> list[list[int]]:
        stride = -(-self.max_requests // 4) * 4
        host = self._chosen_hosts[parity]
        chosen = [host[i * stride:i * stride + bucket].tolist() for i in range(steps)]
        for row in chosen:
            refuse_not_finite(row[:real])       # a row whose logits were not finite (rows that pad the batch are not looked at)
        return chosen

    def _launch_decode_graph(self, ctx: StepContext, bucket: int, steps: int, sampled: bool = False, parity: int = 0, goes_on: bool = False,
                             follows: bool = False) -> None:
        """Queue `steps` decode steps of the prepared batch: a replay of their graph, or, the first time, an eager run
        that is captured on the way.  Nothing is waited for."""
        key = (bucket, length_class(ctx.max_k), steps, sampled) + ((parity, follows) if goes_on else ())
        if self._chosen_devs is None:
            rows = self.MAX_DECODE_STEPS * (-(-self.max_requests // 4) * 4)
            self._chosen_devs = [torch.zeros(rows, dtype=torch.int32, device=self.device) for _ in range(2)]
            self._chosen_hosts = [torch.zeros(rows, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        stride = -(-self.max_requests // 4) * 4                    # rows of 16 bytes and more
        graph = self._graphs.get(key)
        if graph is None or graph[1] != self.arena.generation:
            if graph is not None:
                ops.graph_destroy(graph[0])
                del self._graphs[key]
            self._decode_steps_on_stream(ctx, steps, stride, sampled, parity, goes_on, follows)   # an eager run first: it sizes every scratch buffer
            generation = self.arena.generation
            ops.graph_begin()
            try:
                self._decode_steps_on_stream(ctx, steps, stride, sampled, parity, goes_on, follows)
            finally:
                handle = ops.graph_end()
            if self.arena.generation != generation:
                ops.graph_destroy(handle)
                raise GenerationError("scratch buffers moved during graph capture")
            graph = self._graphs[key] = (handle, generation, None)
            # The eager run above was this launch: its tokens are on their way to the host.  Replaying the graph as
            # well would run every step twice, which keys and values bear (the same values land in the same slots)
            # but a mixer with state of its own does not.
            self.graph_captures += 1
        else:
            ops.graph_launch(graph[0])
            self.graph_replays += 1

    def _decode_steps_on_stream(self, ctx: StepContext, steps: int, stride: int, sampled: bool, parity: int = 0, goes_on: bool = False,
                                follows: bool = False) -> None:
        """goes_on: tokens, positions and lengths are moved on after the last step as well, so that a launch that follows
        this one directly finds its first step's on the device.  follows: this launch is such a one: it begins by
        looking up the cache slots of its first positions, which may lie in pages that the host took for it only
        after the launch before had been queued (their table entries arrive between the two).  parity: which of
        the two result buffers the tokens go to (launches that follow each other take them in turn)."""
        draws = None
        chosen_dev, chosen_host = self._chosen_devs[parity], self._chosen_hosts[parity]
        if sampled:
            temperature, top_p, top_k, draws, seeds = self._sampling_views(ctx.T)
        if follows:
            for group in ctx._groups:
                ops.advance_slots(group.slots, ctx.positions, ctx.token_slot, group.block_table, group.page_size, ctx.counts)
        for i in range(steps):
            ctx.memo.clear()                                       # position tables are made again for the new positions
            h = self.model.forward_hidden(ctx)
            logits = self.model.logits(ctx, h)
            chosen = chosen_dev[i * stride:i * stride + ctx.T]
            if sampled:
                ops.filter_logits(logits, temperature, top_k, top_p)
                ops.choose_tokens(chosen, logits, temperature, seeds, draws, filtered=True)
            else:
                ops.choose_tokens(chosen, logits)
            if i + 1 < steps or goes_on:
                ops.advance_decode(ctx.token_ids, ctx.positions, ctx.token_request, ctx.seq_lens_k, chosen, ctx.counts, draws)
            if i + 1 < steps:
                for group in ctx._groups:
                    ops.advance_slots(group.slots, ctx.positions, ctx.token_slot, group.block_table, group.page_size, ctx.counts)
        ops.copy_to_pinned(chosen_host, chosen_dev, steps * stride)

    # ------------------------------------------------------------------ graphs
    GRAPH_BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128)

    def _graph_bucket(self, entries: Sequence[StepEntry]) -> int:
        """Padded batch size for a decode-only step that may run as a graph, else 0."""
        if not self.use_graph or any(len(e.tokens) != 1 for e in entries):
            return 0
        if torch.cuda.current_stream(self.device).cuda_stream == 0:
            return 0  # the default stream cannot be captured
        # powers of two, and 48 and 96 between them: the kernel for 17..128 rows has forms for 48 and 96 rows, and a
        # layer's four products take 98 us at 48 rows against 101 at 64, 113 at 96 against 132 at 128 (8B sizes)
        bucket = next((b for b in self.GRAPH_BUCKETS if b >= len(entries)), 1 << (len(entries) - 1).bit_length())
        bucket = min(bucket, self.max_requests)
        # A bfloat16 graph of up to 128 rows holds this package's kernels (the few-rows kernels, then the
        # kernel for 17..128 rows); where a shape does not suit that kernel (K no multiple of 256) and the runner
        # may use the vendor library, its products are captured with them.
        most = max(self.kernels.few_rows_max, self.GRAPH_ROWS) if self.dtype == torch.bfloat16 else self.kernels.few_rows_max
        return bucket if bucket <= min(self.max_step_tokens, most) else 0

    def _step_graph(self, entries: Sequence[StepEntry], bucket: int) -> torch.Tensor | None:
        """Replay (capturing first if needed) the graph of a decode step padded to `bucket` rows.

        Logits come back for the wanted rows of the real entries only."""
        ctx = self.prepare(entries, pad_to=bucket)
        key = (bucket, length_class(ctx.max_k))
        graph = self._graphs.get(key)
        if graph is None or graph[1] != self.arena.generation:
            if graph is not None:
                ops.graph_destroy(graph[0])
                del self._graphs[key]
            # an eager run first: it sizes every scratch buffer, so that capture allocates nothing
            h = self.model.forward_hidden(ctx)
            logits = self.model.logits(ctx, h)
            generation = self.arena.generation
            ctx.memo.clear()
            ops.graph_begin()
            try:
                h = self.model.forward_hidden(ctx)
                logits = self.model.logits(ctx, h)
            finally:
                handle = ops.graph_end()
            if self.arena.generation != generation:
                ops.graph_destroy(handle)
                raise GenerationError("scratch buffers moved during graph capture")
            graph = self._graphs[key] = (handle, generation, logits)
            self.graph_captures += 1     # the eager run was this step (see _run_decode_graph): no replay on top of it
        else:
            ops.graph_launch(graph[0])
            self.graph_replays += 1
        wanted = [r for r, entry in enumerate(entries) for _ in entry.want]   # a place asked twice is given twice
        if not wanted:
            return None
        logits = graph[2]
        return logits[:len(entries)] if wanted == list(range(len(entries))) else logits[wanted]

    def drop_graphs(self) -> None:
        """Destroy every captured graph, after the device has finished with them."""
        for key in list(self._plans):
            self._forget_plan(key)
        if self._graphs and self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        for handle, *_ in self._graphs.values():
            ops.graph_destroy(handle)
        self._graphs.clear()
