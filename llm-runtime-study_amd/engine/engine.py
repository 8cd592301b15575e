"""Engine: a loaded model, its cache pool, the step function and the generation entry points.

Reference mini_llm/engine.py:144-352 (`Engine.from_model_dir(...)`, `.generate(...)`,
`.create_scheduler()`, cache accounting, `.synchronize()`); names and defaults of the
options are the reference's.  Differences: the device is the GPU only, `auto` precision is
bfloat16, prompts may be token ids as well as chat messages, and prompts are prefilled in
portions under `max_num_batched_tokens` next to decoding requests.
"""

from __future__ import annotations

import time
from pathlib import Path
from typing import Iterator, Sequence

import torch

from ..cache import CacheManager
from ..errors import EngineError
from ..sampling import Sampler, SamplingConfig
from ..text import TextTokenizer
from ..config import chat_template_for, load_config
from .loading import load_model, random_model, reserve_for, resolve_device, resolve_dtype
from .scheduler import BatchScheduler, GenerationEvent, generate as _generate
from .step import ModelRunner

DEFAULT_PAGE_SIZE = 16
DEFAULT_STEP_TOKENS = 2048


class Engine:
    def __init__(self, config, model, *, device, dtype, max_seq_len: int = 4096, max_batch_size: int = 1,
                 cache_backend: str = "paged", use_cuda_graph: bool = True, page_size: int = DEFAULT_PAGE_SIZE,
                 max_num_batched_tokens: int | None = None, num_pages: int | None = None, tokenizer=None,
                 load_seconds: float = 0.0, library_gemm: bool = True, decode_steps_per_launch: int = 4, kernels=None,
                 use_launch_plans: bool = True, launch_ahead: bool = True):
        if max_batch_size <= 0:
            raise EngineError("max_batch_size must be positive")
        if cache_backend != "paged":
            raise EngineError(f"unsupported cache backend {cache_backend!r}; this runtime has the 'paged' cache only")
        config.validate_context_length(max_seq_len)
        self.config, self.model, self.device, self.dtype = config, model, device, dtype
        self.max_seq_len, self.max_batch_size = max_seq_len, max_batch_size
        self.cache_backend, self.use_cuda_graph = cache_backend, use_cuda_graph
        self.page_size = page_size
        self.max_num_batched_tokens = max(max_batch_size, max_num_batched_tokens or min(DEFAULT_STEP_TOKENS, max_seq_len))
        self.num_pages = num_pages
        # greedy decoding runs up to this many steps from one graph launch (1: the host sees every step)
        self.decode_steps_per_launch = decode_steps_per_launch
        # which matrix-product kernels the steps use (kernels.ops.KernelChoice); unless given: the vendor library
        # for bfloat16 products of many rows if `library_gemm`, this package's own kernels for everything else
        self.kernels = kernels
        self.library_gemm = library_gemm if kernels is None else kernels.library
        # steps outside graphs are recorded once per shape and made again from the record (see engine/step.py)
        self.use_launch_plans = use_launch_plans
        # decode launches are queued one ahead: the device never waits for the host between them (see BatchScheduler)
        self.launch_ahead = launch_ahead
        self.tokenizer = tokenizer
        self.load_seconds = load_seconds
        self.quantization = "dense"
        self.stream = torch.cuda.Stream(device)
        self._reload = None        # makes the model again in another dtype: set by from_model_dir / from_config
        self._runner: ModelRunner | None = None
        self._sampler = Sampler(device)

    # ---------------------------------------------------------------- loading
    @classmethod
    def from_model_dir(cls, model_dir, *, device="auto", dtype="auto", max_seq_len: int = 4096, max_batch_size: int = 1,
                       cache_backend: str = "paged", use_cuda_graph: bool = True, stored_precision: bool = False,
                       **options) -> "Engine":
        """Load config.json and the safetensors weights of `model_dir` onto the GPU.  The tensors must be
        stored in the configuration's `torch_dtype` unless `stored_precision` is set (see load_model)."""
        started = time.perf_counter()
        config = load_config(model_dir)
        config.validate_context_length(max_seq_len)
        selected_device, selected_dtype = resolve_device(device), resolve_dtype(dtype)
        cls._reserve(config, selected_dtype, selected_device, max_seq_len, max_batch_size, options)
        config, model = load_model(model_dir, selected_dtype, selected_device, config, stored_precision)
        tokenizer = TextTokenizer.from_model_dir(model_dir, config.vocab_size, chat_template_for(config))
        engine = cls(config, model, device=selected_device, dtype=selected_dtype, max_seq_len=max_seq_len,
                     max_batch_size=max_batch_size, cache_backend=cache_backend, use_cuda_graph=use_cuda_graph,
                     tokenizer=tokenizer, **options)
        engine._reload = lambda dtype: load_model(model_dir, dtype, selected_device, config, stored_precision)[1]
        engine.synchronize()
        engine.load_seconds = time.perf_counter() - started
        return engine

    @classmethod
    def from_config(cls, config, *, seed: int = 0, init: str = "normal", device="auto", dtype="auto", **options) -> "Engine":
        """Random weights made on the device for `config` (a typed configuration)."""
        started = time.perf_counter()
        selected_device, selected_dtype = resolve_device(device), resolve_dtype(dtype)
        cls._reserve(config, selected_dtype, selected_device, options.get("max_seq_len", 4096), options.get("max_batch_size", 1), options)
        model = random_model(config, seed, selected_dtype, selected_device, init)
        engine = cls(config, model, device=selected_device, dtype=selected_dtype, **options)
        engine._reload = lambda dtype: random_model(config, seed, dtype, selected_device, init)
        engine.synchronize()
        engine.load_seconds = time.perf_counter() - started
        return engine

    @staticmethod
    def _pool_pages(num_pages, max_seq_len: int, page_size: int, max_batch_size: int) -> int:
        return num_pages or -(-max_seq_len // page_size) * max_batch_size

    @classmethod
    def _reserve(cls, config, dtype, device, max_seq_len: int, max_batch_size: int, options: dict) -> None:
        """One segment of device memory for the weights, the cache pool and the step's buffers of the engine that
        is about to be made (see engine/loading.py); `reserve_memory=False` among the options leaves it out."""
        if not options.pop("reserve_memory", True) or max_batch_size <= 0:
            return
        page_size = options.get("page_size", DEFAULT_PAGE_SIZE)
        reserve_for(config, dtype, device, page_size, cls._pool_pages(options.get("num_pages"), max_seq_len, page_size, max_batch_size))

    # ------------------------------------------------------------------ cache
    @property
    def runner(self) -> ModelRunner:
        """The step function over this engine's cache pool, made on first use: the pool holds
        max_seq_len * max_batch_size tokens unless `num_pages` says otherwise."""
        if self._runner is None:
            pages = self._pool_pages(self.num_pages, self.max_seq_len, self.page_size, self.max_batch_size)
            cache = CacheManager(self.model.cache_needs(), page_size=self.page_size, num_pages=pages,
                                 max_requests=self.max_batch_size, max_seq_len=self.max_seq_len,
                                 dtype=self.dtype, device=self.device)
            self._runner = ModelRunner(self.model, cache, max_step_tokens=self.max_num_batched_tokens,
                                       dtype=self.dtype, device=self.device, use_graph=self.use_cuda_graph,
                                       library_gemm=self.library_gemm, kernels=self.kernels, use_plans=self.use_launch_plans)
        return self._runner

    @property
    def cache_manager(self) -> CacheManager:
        return self.runner.cache

    @property
    def last_cache_capacity(self) -> int:
        return self.cache_manager.last_allocation_tokens

    @property
    def last_cache_num_bytes(self) -> int:
        return self.cache_manager.last_allocation_tokens * self.cache_manager.bytes_per_token()

    # ------------------------------------------------------------- generation
    def create_scheduler(self, ignore_eos: bool = False) -> BatchScheduler:
        """A continuous-batching scheduler over this engine's cache and step function; with
        `ignore_eos` requests run to their length limits (benchmarks with random weights)."""
        return BatchScheduler(
            self.runner, self._sampler, max_batch_size=self.max_batch_size, max_seq_len=self.max_seq_len,
            max_step_tokens=self.max_num_batched_tokens, eos_token_ids=() if ignore_eos else self.config.eos_token_ids,
            vocab_size=self.config.vocab_size, tokenizer=self.tokenizer, synchronize=self.synchronize,
            decode_steps_per_launch=self.decode_steps_per_launch if self.use_cuda_graph else 1, launch_ahead=self.launch_ahead)

    def generate(self, message_batches: Sequence, *, max_new_tokens: int, sampling: SamplingConfig = SamplingConfig(),
                 enable_thinking: bool = False, ignore_eos: bool = False) -> Iterator[tuple[int, GenerationEvent]]:
        """Events (request index, GenerationEvent) of the given prompts, each a list of ChatMessage
        or of token ids; requests beyond max_batch_size wait for a free slot."""
        scheduler = self.create_scheduler(ignore_eos)
        inner = _generate(scheduler, message_batches, max_new_tokens=max_new_tokens, sampling=sampling,
                          enable_thinking=enable_thinking)

        def on_stream():
            try:
                while True:
                    with torch.cuda.device(self.device), torch.cuda.stream(self.stream):
                        try:
                            item = next(inner)
                        except StopIteration:
                            return
                    yield item
            finally:
                inner.close()

        return on_stream()

    def generate_tokens(self, prompts: Sequence[Sequence[int]], *, max_new_tokens: int,
                        sampling: SamplingConfig = SamplingConfig(), ignore_eos: bool = False) -> list[list[int]]:
        """Token ids generated for each prompt (a convenience over generate())."""
        out = [[] for _ in prompts]
        for index, event in self.generate([list(p) for p in prompts], max_new_tokens=max_new_tokens, sampling=sampling,
                                          ignore_eos=ignore_eos):
            if event.token_id is not None:
                out[index].append(event.token_id)
        return out

    def allocate_cache(self, capacity: int):
        """A request's cache with `capacity` tokens promised to it (reference Engine.allocate_cache,
        mini_llm/engine.py:298-299): for callers that drive the step function themselves."""
        if capacity <= 0 or capacity > self.max_seq_len:
            raise EngineError(f"cache capacity must be within 1..{self.max_seq_len}, got {capacity}")
        manager = self.cache_manager
        if not manager.can_admit(capacity):
            raise EngineError(f"the KV cache cannot promise {capacity} more tokens")
        return manager.admit(reserve_tokens=capacity)

    def release_cache(self, cache) -> None:
        """Give a cache from allocate_cache() back (mini_llm/engine.py:301-302); idempotent."""
        self.cache_manager.release(cache)

    def to(self, *, device=None, dtype=None) -> "Engine":
        """The same engine in another precision (reference Engine.to, mini_llm/engine.py:304-346).  The
        weights are made again from their source (the model folder, or the configuration and seed)
        rather than converted in place, so float32 after bfloat16 has the checkpoint's precision;
        cache pool, graphs and step function are rebuilt on next use.  The device cannot change."""
        if device is not None and resolve_device(device) != self.device:
            raise EngineError(f"this runtime has one device, {self.device}; it cannot move to {device}")
        selected = self.dtype if dtype is None else resolve_dtype(dtype)
        if selected == self.dtype:
            return self
        if self._runner is not None and self._runner.cache.active_requests:
            raise EngineError("cannot move an engine while request caches are active")
        if self._reload is None:
            raise EngineError("this engine was not made by from_model_dir or from_config and cannot make its weights again")
        if self._runner is not None:
            self._runner.drop_graphs()
            self._runner = None
        self.model = None                  # the old weights go before the new ones come
        self.model = self._reload(selected)
        self.dtype = selected
        self.synchronize()
        return self

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)
