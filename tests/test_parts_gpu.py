"""Each part alone against its plain function, and the generality of the layer description:
a layer run twice, a layer reading another layer's cache, a windowed layer whose pages are
given back, and a toy mixer with state of its own that is registered from here."""

import math

import numpy as np
import pytest
import torch

from tests.plain import model as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def close(got, want, dtype, f32=2e-5, bf16=3e-2):
    if dtype == torch.float32:
        torch.testing.assert_close(got.double().cpu(), want.double(), rtol=f32, atol=f32)
    else:
        err = (got.double().cpu() - want.double()).norm() / want.double().norm()
        assert err < bf16, f"relative error {err:.3g}"


def build_runner(spec, weights, dtype, *, page_size=16, num_pages=64, max_requests=4, max_seq_len=512, max_step_tokens=512, use_graph=False):
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.engine.step import ModelRunner
    from llm_runtime_study_amd.models import DecoderModel

    model = DecoderModel(spec)
    model.bind({k: v.to("cuda") for k, v in weights.items()}, dtype)
    cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         max_seq_len=max_seq_len, dtype=dtype, device="cuda")
    return ModelRunner(model, cache, max_step_tokens=max_step_tokens, dtype=dtype, device="cuda", use_graph=use_graph)


def spec_and_weights(raw, seed, edit=None):
    """ModelSpec of a Qwen3 configuration (optionally edited) and random weights for it."""
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.weights import random_tensors

    spec = spec_for(config_from_dict(raw))
    if edit is not None:
        spec = edit(spec)
    weights = random_tensors(DecoderModel(spec).tensors(), seed, torch.bfloat16, "scaled")
    return spec, weights


class PartHarness:
    """A step context around one part: a runner whose model is never run."""

    def __init__(self, needs, dtype, page_size=16, max_step_tokens=256):
        from llm_runtime_study_amd.cache import CacheManager
        from llm_runtime_study_amd.engine.step import ModelRunner

        class NoModel:
            def graph_safe(self):
                return False

        self.cache = CacheManager(needs, page_size=page_size, num_pages=max(32, max_step_tokens // page_size + 1), max_requests=4,
                                  max_seq_len=max_step_tokens, dtype=dtype, device="cuda")
        self.runner = ModelRunner(NoModel(), self.cache, max_step_tokens=max_step_tokens, dtype=dtype, device="cuda")

    def context(self, entries):
        from llm_runtime_study_amd.engine.step import StepEntry

        step = []
        for request, tokens in entries:
            self.cache.extend(request, len(tokens))
            step.append(StepEntry(request, tokens, []))
        return self.runner.prepare(step)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("norm", PartSpec("rmsnorm", {"size": 96, "eps": 1e-5}))
    weight = (1 + 0.1 * torch.randn(96)).to(torch.bfloat16)
    part.bind({"weight": weight.cuda()}, dtype)
    harness = PartHarness([], dtype)
    ctx = harness.context([(harness.cache.admit("a"), [1] * 7)])
    h = torch.randn(7, 96)
    close(part.forward(ctx, h.cuda()), plain.rms_norm(h, weight.float(), 1e-5), dtype, bf16=1e-2)
    rows = torch.tensor([6, 2], dtype=torch.int32, device="cuda")
    close(part.forward(ctx, h.cuda(), rows=rows, count=2), plain.rms_norm(h[[6, 2]], weight.float(), 1e-5), dtype, bf16=1e-2)


def test_rotary_part_tables_are_made_once_per_step():
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("position", PartSpec("rope_half", {"rotary_dim": 32, "theta": 1e6}))
    harness = PartHarness([], torch.float32)
    a, b = harness.cache.admit("a"), harness.cache.admit("b")
    harness.context([(a, [1] * 20)])
    ctx = harness.context([(a, [1] * 3), (b, [1] * 5)])     # positions 20..22 and 0..4
    cos, sin = part.tables(ctx)
    assert part.tables(ctx)[0].data_ptr() == cos.data_ptr()
    want_cos, want_sin = plain.rope_tables(torch.tensor([20, 21, 22, 0, 1, 2, 3, 4]), 32, 1e6)
    torch.testing.assert_close(cos.cpu(), want_cos[:, :16], rtol=0, atol=1e-6)
    torch.testing.assert_close(sin.cpu(), want_sin[:, :16], rtol=0, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part_adds_into_the_residual(dtype):
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("feed_forward", PartSpec("swiglu", {"hidden_size": 96, "intermediate_size": 160}))
    w = {n: (torch.randn(s) / math.sqrt(s[1])).to(torch.bfloat16) for n, s in
         (("gate_proj.weight", (160, 96)), ("up_proj.weight", (160, 96)), ("down_proj.weight", (96, 160)))}
    part.bind({k: v.cuda() for k, v in w.items()}, dtype)
    harness = PartHarness([], dtype)
    ctx = harness.context([(harness.cache.admit("a"), [1] * 9)])
    x = torch.randn(9, 96).to(dtype)
    residual = torch.randn(9, 96)
    out = residual.clone().cuda()
    part.forward(ctx, x.cuda(), out)
    want = residual + plain.swiglu(x.float(), *(w[n].float() for n in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    close(out, want, dtype, bf16=1e-2)


def test_swiglu_part_of_a_prompt_portion_divides_the_long_k_of_its_second_product():
    """300 rows, 1,024 wide, 4,096 between: the second product has 16 tiles of 256 x 128 for 256 compute units and a
    K four times its width, so it goes to this package's kernel with K in 8 parts (the first one to the library)."""
    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.parts import PartSpec, create
    from llm_runtime_study_amd.parts.linear import plan

    hidden, inter, rows = 1024, 4096, 300
    if ops.compute_units() == 256:
        assert ops.gemm_lines_splits(rows, hidden, inter) == 8
        assert plan(rows, hidden, inter, weight_dtype=torch.bfloat16, run_dtype=torch.bfloat16, out_dtype=torch.float32,
                    arrives="tensor", accumulate=True)[0] == "own"
    part = create("feed_forward", PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter}))
    g = torch.Generator().manual_seed(31)
    w = {n: (torch.randn(s, generator=g) / math.sqrt(s[1])).to(torch.bfloat16) for n, s in
         (("gate_proj.weight", (inter, hidden)), ("up_proj.weight", (inter, hidden)), ("down_proj.weight", (hidden, inter)))}
    part.bind({k: v.cuda() for k, v in w.items()}, torch.bfloat16)
    harness = PartHarness([], torch.bfloat16, max_step_tokens=512)
    ctx = harness.context([(harness.cache.admit("a"), [1] * rows)])
    x = torch.randn(rows, hidden, generator=g).to(torch.bfloat16)
    residual = torch.randn(rows, hidden, generator=g)
    out = residual.clone().cuda()
    part.forward(ctx, x.cuda(), out)
    want = residual + plain.swiglu(x.float(), *(w[n].float() for n in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    close(out, want, torch.bfloat16, bf16=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,bias,window", [(4, 2, 16, False, None), (6, 3, 48, True, None), (8, 2, 32, True, 9)])
def test_attention_part_in_portions_matches_whole_sequence(dtype, nq, nkv, d, bias, window):
    from llm_runtime_study_amd.parts import PartSpec, create

    hidden, t = 80, 37
    params = {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d, "qk_norm": True, "qk_norm_eps": 1e-5,
              "bias": bias, "window": window, "position": PartSpec("rope_half", {"rotary_dim": d, "theta": 1e4})}
    part = create("mixer", PartSpec("gqa_attention", params))
    g = torch.Generator().manual_seed(3)
    w = {}
    for name, spec in part.tensors().items():
        if spec.role == "norm":
            w[name] = (1 + 0.1 * torch.randn(spec.shape, generator=g)).to(torch.bfloat16)
        elif spec.role == "bias":
            w[name] = (0.1 * torch.randn(spec.shape, generator=g)).to(torch.bfloat16)
        else:
            w[name] = (torch.randn(spec.shape, generator=g) / math.sqrt(spec.shape[1])).to(torch.bfloat16)
    part.bind({k: v.cuda() for k, v in w.items()}, dtype)
    x = torch.randn(t, hidden, generator=g).to(dtype)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rms_norm_eps=1e-5, rope_theta=1e4)
    want, _ = plain.qwen3_attention(x.double(), {f"a.{k}": v.double() for k, v in w.items()}, "a", cfg, torch.arange(t), window)

    harness = PartHarness([part.cache_need()], dtype, page_size=4)
    request = harness.cache.admit("a")
    got = torch.zeros(t, hidden, device="cuda")
    at = 0
    for n in (5, 1, 11, 2, 1, 17):       # portions that start and end inside pages
        ctx = harness.context([(request, [1] * n)])
        part.forward(ctx, x[at:at + n].cuda(), got[at:at + n], harness.cache.layer_caches[0])
        harness.cache.trim(request)
        at += n
    close(got, want, dtype)
    if window is not None:
        assert request.first_live[0] > 0     # pages behind the window went back to the pool


@pytest.mark.parametrize("dtype", DTYPES)
def test_layer_run_twice_and_layer_reading_another_cache(dtype):
    """Schedule [0, 1, 1, 2<-0]: layer 1 runs twice with a cache for each run; layer 2 owns no keys
    or values and attends to what the first entry cached."""
    from llm_runtime_study_amd.models import ScheduleEntry
    from llm_runtime_study_amd.parts import PartSpec
    from tests.helpers import TINY_B
    import dataclasses

    def edit(spec):
        block = spec.layers[0]
        shared_mixer = PartSpec("gqa_attention", dict(block.params["mixer"].params, kv_shared=True))
        shared = PartSpec("prenorm", dict(block.params, mixer=shared_mixer))
        return dataclasses.replace(spec, layers=(block, block, shared),
                                   schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(2, cache_from=0)))

    spec, weights = spec_and_weights(TINY_B, 21, edit)
    assert "model.layers.2.self_attn.k_proj.weight" not in weights
    runner = build_runner(spec, weights, dtype)
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].entries == [0, 1, 2]
    ids = np.random.default_rng(0).integers(0, TINY_B["vocab_size"], 45).tolist()
    want = plain.qwen3_forward({k: v.double() for k, v in weights.items()}, TINY_B, ids, schedule=[0, 1, 1, 2], kv_from={3: 0})
    from llm_runtime_study_amd.engine.step import StepEntry

    request = runner.cache.admit("a")
    rows, at = [], 0
    for n in (20, 1, 1, 9, 2, 12):
        rows.append(runner.step([StepEntry(request, ids[at:at + n], list(range(n)))]).clone())
        at += n
    close(torch.cat(rows), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_windowed_layers_beside_full_ones_give_pages_back(dtype):
    """Layers 0 and 2 see a window of 24 positions, layer 1 everything: two cache groups with pools
    of their own; the windowed group's pool is far too small for the whole sequence."""
    from llm_runtime_study_amd.parts import PartSpec
    from tests.helpers import TINY_B
    import dataclasses

    def edit(spec):
        block = spec.layers[0]
        windowed = PartSpec("prenorm", dict(block.params, mixer=PartSpec("gqa_attention", dict(block.params["mixer"].params, window=24))))
        return dataclasses.replace(spec, layers=(windowed, block, windowed))

    spec, weights = spec_and_weights(TINY_B, 22, edit)
    runner = build_runner(spec, weights, dtype, page_size=8, num_pages=40)
    assert [g.entries for g in runner.cache.groups] == [[0, 2], [1]]
    ids = np.random.default_rng(1).integers(0, TINY_B["vocab_size"], 300).tolist()
    want = plain.qwen3_forward({k: v.double() for k, v in weights.items()}, TINY_B, ids, windows={0: 24, 2: 24})
    from llm_runtime_study_amd.engine.step import StepEntry

    request = runner.cache.admit("a")
    rows, at, peak = [], 0, 0
    sizes = [30, 1, 1, 2, 17, 40, 1, 1, 1, 8] * 6
    for n in sizes:
        n = min(n, len(ids) - at)
        if n == 0:
            break
        rows.append(runner.step([StepEntry(request, ids[at:at + n], list(range(n)))]).clone())
        at += n
        peak = max(peak, runner.cache.used_pages(0))
    close(torch.cat(rows), want, dtype)
    assert runner.cache.used_pages(1) == -(-300 // 8)        # the full group holds every page
    assert peak <= 10 and runner.cache.used_pages(0) <= 4     # the windowed group a handful, reused many times
    runner.cache.check_invariants()


class RunningMeanMixer:
    """Toy mixer with state of its own, defined here and unknown to the framework: the output at a
    token is W applied to the mean of all inputs of the request up to and including that token.
    State per request: the running sum [H] and the count."""

    def __init__(self, hidden_size: int):
        from llm_runtime_study_amd.parts import TensorSpec
        self.hidden_size = hidden_size
        self._spec = TensorSpec((hidden_size, hidden_size))
        self.weight = None

    def tensors(self):
        return {"mix.weight": self._spec}

    def bind(self, weights, dtype):
        self.weight = weights["mix.weight"].float()

    def weight_bytes(self):
        return 0

    def cache_need(self):
        from llm_runtime_study_amd.parts import StateNeed
        return StateNeed((self.hidden_size + 1,), torch.float32)

    def forward(self, ctx, x, residual, cache):
        start = 0
        for n, slot in zip(ctx.host_q_lens, ctx.host_slots):
            state = cache.state[slot]
            sums = state[:-1] + torch.cumsum(x[start:start + n].float(), 0)
            counts = state[-1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            residual[start:start + n] += (sums / counts[:, None]) @ self.weight.T
            state[:-1] = sums[-1]
            state[-1] = counts[-1]
            start += n


def plain_running_mean_model(weights, cfg, ids, layers):
    h = weights["model.embed_tokens.weight"][torch.as_tensor(ids)]
    for i in range(layers):
        p = f"model.layers.{i}"
        x = plain.rms_norm(h, weights[f"{p}.input_layernorm.weight"], cfg["rms_norm_eps"])
        mean = torch.cumsum(x, 0) / torch.arange(1, len(ids) + 1, dtype=x.dtype)[:, None]
        h = h + mean @ weights[f"{p}.mixer.mix.weight"].T
        x = plain.rms_norm(h, weights[f"{p}.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        h = h + plain.swiglu(x, weights[f"{p}.mlp.gate_proj.weight"], weights[f"{p}.mlp.up_proj.weight"], weights[f"{p}.mlp.down_proj.weight"])
    h = plain.rms_norm(h, weights["model.norm.weight"], cfg["rms_norm_eps"])
    return h @ weights["lm_head.weight"].T


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_is_registered_built_and_stepped(dtype):
    """In bfloat16 the steps of at most 16 rows also show that a part which knows nothing of the
    norm hand-overs between matrix products is simply given normalised rows."""
    from llm_runtime_study_amd.engine.step import StepEntry
    from llm_runtime_study_amd.models import DecoderModel, ModelSpec, ScheduleEntry
    from llm_runtime_study_amd.parts import PartSpec, register
    from llm_runtime_study_amd.weights import random_tensors

    register("mixer", "toy_running_mean", RunningMeanMixer)
    hidden, vocab, eps = 48, 97, 1e-5
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    block = PartSpec("prenorm", {
        "mixer": PartSpec("toy_running_mean", {"hidden_size": hidden}),
        "feed_forward": PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 80}),
        "mixer_norm": norm, "ff_norm": norm,
        "names": {"mixer": "mixer", "feed_forward": "mlp", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"},
    })
    spec = ModelSpec(architecture="ToyRunningMean", vocab_size=vocab, hidden_size=hidden, layers=(block, block),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm, max_positions=256)
    weights = random_tensors(DecoderModel(spec).tensors(), 5, torch.bfloat16, "scaled")
    runner = build_runner(spec, weights, dtype)
    assert not runner.use_graph and len(runner.cache.state_entries) == 2 and not runner.cache.groups
    rng = np.random.default_rng(2)
    requests = {k: rng.integers(0, vocab, n).tolist() for k, n in (("a", 40), ("b", 23), ("c", 31))}
    double = {k: v.double() for k, v in weights.items()}
    want = {k: plain_running_mean_model(double, {"rms_norm_eps": eps}, ids, 2) for k, ids in requests.items()}
    # a and b interleaved in portions and single tokens; c reuses a's slot after a ends
    caches = {k: None for k in requests}
    progress = {k: 0 for k in requests}
    plan = [{"a": 7, "b": 1}, {"a": 1, "b": 9}, {"b": 2}, {"a": 20, "b": 1}, {"a": 12, "b": 10}, {"c": 30}, {"c": 1}]
    got = {k: [] for k in requests}
    for step in plan:
        entries = []
        for key, n in step.items():
            if caches[key] is None:
                caches[key] = runner.cache.admit(key)
            at = progress[key]
            entries.append(StepEntry(caches[key], requests[key][at:at + n], list(range(n))))
            progress[key] = at + n
        logits = runner.step(entries)
        row = 0
        for key, n in step.items():
            got[key].append(logits[row:row + n].clone())
            row += n
            if progress[key] == len(requests[key]):
                runner.cache.release(caches[key])
    assert caches["c"].slot == caches["a"].slot
    for key in requests:
        close(torch.cat(got[key]), want[key], dtype, f32=1e-4)


class GraphSafeRunningMean(RunningMeanMixer):
    """The same toy mixer, able to run inside a captured decode step: there it finds its state rows through
    the slot ids on the device (a replay sees the slots of its own step, and the rows that pad the batch
    point at the trash slot), works in place on scratch buffers and leaves the product to the package."""

    graph_safe = True

    def bind(self, weights, dtype):
        super().bind(weights, dtype)
        self.weight_run = weights["mix.weight"].to(dtype).contiguous()

    def forward(self, ctx, x, residual, cache):
        from llm_runtime_study_amd.parts.linear import linear

        if not ctx.all_decode:
            return super().forward(ctx, x, residual, cache)
        rows_n, hidden = ctx.T, self.hidden_size
        index = ctx.scratch("toy_index", (rows_n,), torch.int64)
        index.copy_(ctx.slot_ids)
        rows = ctx.scratch("toy_rows", (rows_n, hidden + 1), torch.float32)
        torch.index_select(cache.state, 0, index, out=rows)
        rows[:, :-1].add_(x)
        rows[:, -1].add_(1.0)
        mean32 = ctx.scratch("toy_mean32", (rows_n, hidden), torch.float32)
        torch.div(rows[:, :-1], rows[:, -1:], out=mean32)
        mean = ctx.scratch("toy_mean", (rows_n, hidden), ctx.dtype)
        mean.copy_(mean32)
        linear(ctx, residual, mean, self.weight_run, accumulate=True)
        cache.state.index_copy_(0, index, rows)


def toy_state_model(kind, cls):
    from llm_runtime_study_amd.models import DecoderModel, ModelSpec, ScheduleEntry
    from llm_runtime_study_amd.parts import PartSpec, register
    from llm_runtime_study_amd.weights import random_tensors

    register("mixer", kind, cls)
    hidden, vocab, eps = 48, 97, 1e-5
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    block = PartSpec("prenorm", {
        "mixer": PartSpec(kind, {"hidden_size": hidden}),
        "feed_forward": PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 80}),
        "mixer_norm": norm, "ff_norm": norm,
        "names": {"mixer": "mixer", "feed_forward": "mlp", "mixer_norm": "input_layernorm", "ff_norm": "post_attention_layernorm"},
    })
    spec = ModelSpec(architecture="ToyRunningMean", vocab_size=vocab, hidden_size=hidden, layers=(block, block),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm, max_positions=256)
    weights = random_tensors(DecoderModel(spec).tensors(), 5, torch.bfloat16, "scaled")
    return spec, weights, vocab, eps


@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_that_pad_a_graph_batch_leave_every_request_state_alone(dtype):
    """Three requests decode as a captured batch of four rows: the fourth row belongs to no request.  Its
    state goes to the trash slot, so the request in slot 0 keeps its own."""
    from llm_runtime_study_amd.engine.step import StepEntry

    spec, weights, vocab, eps = toy_state_model("toy_running_mean_graph", GraphSafeRunningMean)
    runner = build_runner(spec, weights, dtype, use_graph=True)
    assert runner.use_graph
    cache = runner.cache
    assert cache.layer_caches[0].state.shape == (cache.max_requests + 1, 49) and cache.trash_slot == cache.max_requests
    rng = np.random.default_rng(3)
    requests = {k: rng.integers(0, vocab, n).tolist() for k, n in (("a", 18), ("b", 13), ("c", 20))}
    double = {k: v.double() for k, v in weights.items()}
    want = {k: plain_running_mean_model(double, {"rms_norm_eps": eps}, ids, 2) for k, ids in requests.items()}
    prompt = {"a": 10, "b": 5, "c": 12}
    got = {k: [] for k in requests}
    with torch.cuda.stream(torch.cuda.Stream("cuda")):
        caches = {k: cache.admit(k) for k in requests}
        assert caches["a"].slot == 0
        runner.step([StepEntry(caches[k], requests[k][:n], []) for k, n in prompt.items()])
        for step in range(8):
            logits = runner.step([StepEntry(caches[k], [requests[k][prompt[k] + step]], [0]) for k in requests])
            for row, k in enumerate(requests):
                got[k].append(logits[row].clone())
        torch.cuda.synchronize()
        assert runner.graph_captures == 1 and runner.graph_replays == 7       # the capturing step runs once, eagerly
        trash = cache.layer_caches[0].state[cache.trash_slot]
        assert trash[-1].item() > 0          # the padding row counted its tokens there
        runner.drop_graphs()
    for k in requests:
        close(torch.stack(got[k]), want[k][prompt[k]:prompt[k] + 8], dtype, f32=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_failing_step_puts_per_request_state_back(dtype):
    """The mixers of both layers have moved their state on when the second layer's feed-forward raises:
    the rows of the step's requests are as before, and the step run again gives the right logits."""
    from llm_runtime_study_amd.engine.step import StepEntry

    spec, weights, vocab, eps = toy_state_model("toy_running_mean", RunningMeanMixer)
    runner = build_runner(spec, weights, dtype)
    cache = runner.cache
    rng = np.random.default_rng(4)
    ids = {k: rng.integers(0, vocab, 24).tolist() for k in ("a", "b")}
    double = {k: v.double() for k, v in weights.items()}
    want = {k: plain_running_mean_model(double, {"rms_norm_eps": eps}, v, 2) for k, v in ids.items()}
    caches = {k: cache.admit(k) for k in ids}
    runner.step([StepEntry(caches["a"], ids["a"][:9], []), StepEntry(caches["b"], ids["b"][:16], [])])
    states = [cache.layer_caches[i].state.clone() for i in (0, 1)]
    entries = [StepEntry(caches["a"], ids["a"][9:], list(range(15))), StepEntry(caches["b"], ids["b"][16:17], [0])]
    feed_forward = runner.model.layers[1].feed_forward
    original = feed_forward.forward

    def broken(*args, **kwargs):
        raise RuntimeError("the feed-forward fails")

    feed_forward.forward = broken
    with pytest.raises(RuntimeError, match="feed-forward fails"):
        runner.step(entries)
    feed_forward.forward = original
    assert [caches[k].length for k in ids] == [9, 16]
    for i in (0, 1):
        assert torch.equal(cache.layer_caches[i].state, states[i])
    logits = runner.step(entries)
    close(logits[:15], want["a"][9:], dtype, f32=1e-4)
    close(logits[15:], want["b"][16:17], dtype, f32=1e-4)
