"""Host-side choices that kernels are launched with: they must not change from step to step in a way
that would make an eager step and a captured graph disagree, and must respect what a kernel can hold."""

from llm_runtime_study_amd.parts.attention import GQAAttention
from llm_runtime_study_amd.parts.base import length_class


def test_length_class_is_256_times_a_power_of_two():
    assert [length_class(n) for n in (0, 1, 255, 256, 511, 512, 1023, 1024, 3000, 4096, 40000)] == \
        [0, 0, 0, 256, 256, 512, 512, 1024, 2048, 4096, 32768]
    for n in range(1, 5000, 37):
        c = length_class(n)
        assert c <= n and (c == 0 or (n < 2 * c and (c // 256) & (c // 256 - 1) == 0))


def test_decode_splits_follow_the_class_not_the_length(monkeypatch):
    from llm_runtime_study_amd.kernels import ops

    monkeypatch.setattr(ops, "compute_units", lambda: 256)
    splits = GQAAttention._decode_splits
    # short contexts and large batches: one workgroup per (token, kv head)
    assert splits(64, 100, 4096, 16) == 1 and splits(512, 5000, 8192, 16) == 1
    # few rows, long context: more workgroups, at least 256 keys each
    assert splits(8, 2048, 4096, 16) == 8 and splits(8, 2049, 4096, 16) == 8 and splits(8, 4095, 4096, 16) == 8
    assert splits(8, 4096, 8192, 16) == 16 and splits(64, 2048, 4096, 16) == 8 and splits(128, 2048, 4096, 16) == 4
    # five workgroups for every eight compute units, or more: not divided
    assert splits(152, 2048, 4096, 16) == 4 and splits(160, 2048, 4096, 16) == 1 and splits(192, 8192, 8192, 16) == 1
    # between one and one and a half workgroups a unit, from 2,048 tokens of context on: two parts
    assert splits(256, 4000, 4096, 16) == 1 and splits(264, 4000, 4096, 16) == 2 and splits(384, 2048, 4096, 16) == 2
    assert splits(385, 4000, 4096, 16) == 1 and splits(384, 2047, 4096, 16) == 1 and splits(512, 4000, 4096, 16) == 1
    for workgroups in (1, 8, 24, 64, 200, 300):
        for length in range(1, 20000, 501):
            n = splits(workgroups, length, 32768, 16)
            assert n == splits(workgroups, max(length_class(length), 1), 32768, 16)   # the same all over a class
            assert 1 <= n <= 64 and (n == 1 or length // n >= 256)


def test_decode_splits_keep_a_workgroups_block_table_inside_lds(monkeypatch):
    from llm_runtime_study_amd.kernels import ops

    monkeypatch.setattr(ops, "compute_units", lambda: 256)
    splits = GQAAttention._decode_splits
    # one workgroup can hold 4,096 block table entries: contexts beyond that are split even when the batch is large
    assert splits(512, 100, 4096 * 16, 16) == 1
    assert splits(512, 100, 4096 * 16 + 1, 16) == 2
    assert splits(512, 100, 1 << 20, 16) == 16
    assert splits(512, 100, 1 << 20, 64) == 4


def test_prefill_splits_only_where_groups_leave_the_chip_idle(monkeypatch):
    from llm_runtime_study_amd.kernels import ops

    monkeypatch.setattr(ops, "compute_units", lambda: 256)
    splits = GQAAttention._prefill_splits
    assert splits(1024, 100000, 1 << 20) == 1           # enough groups already (a 2,048-token prompt, 8 kv heads)
    assert splits(512, 1024, 1 << 20) == 1              # short contexts
    assert splits(256, 33216, 1 << 20) == 8             # a 512-token portion after 32,704 tokens
    assert splits(32, 32768, 1 << 20) == 32             # a 64-token portion
    assert splits(8, 32768, 1 << 16) == 32              # one token: as many as allowed
    assert splits(8, 1 << 20, 16 << 20) == 4            # partial results stay within 256 MB
    # contexts under 16,384 tokens: towards two workgroups a unit, at least 256 keys each, none from two a unit on
    assert splits(8, 2048, 1 << 16) == 8 and splits(32, 2064, 1 << 20) == 8 and splits(128, 2048, 1 << 20) == 4
    assert splits(256, 2048, 1 << 20) == 2 and splits(256, 4096, 1 << 20) == 2 and splits(1016, 2047, 1 << 20) == 1
    assert splits(64, 700, 1 << 20) == 2                # 256 keys each
    # and only where the longest context is four times the step's tokens or more: the merge costs by the token
    assert splits(256, 2048, 1 << 20, 4, 512) == 2 and splits(256, 2047, 1 << 20, 4, 512) == 1 and splits(256, 512, 1 << 20, 4, 512) == 1
    assert splits(64, 700, 1 << 20, 4, 128) == 2 and splits(64, 384, 1 << 20, 4, 128) == 1
    assert splits(256, 33216, 1 << 20, 4, 16384) == 8   # not a rule for long contexts
    # kv groups of five to eight heads (one walk with a wave a head): one workgroup a unit is the aim
    assert splits(256, 8192, 1 << 20, 5) == 1 and splits(128, 2048, 1 << 20, 5) == 2 and splits(32, 2064, 1 << 20, 8) == 8
    assert splits(512, 2048, 1 << 20, 5) == 1 and splits(256, 33216, 1 << 20, 5) == 8 and splits(512, 33216, 1 << 20, 5) == 1


def test_query_groups_of_32_behind_long_contexts():
    """`lrs_attention_prefill_group_for`: 16 queries a group for fresh prompts up to 2,048 tokens, 32 beyond, and 32
    already for portions of 2,048 (1,024) tokens whose context is twice (four times) as long."""
    from llm_runtime_study_amd.kernels import ops

    if ops.compute_units() not in (0, 256):
        return
    group = ops.attention_prefill_group
    assert group(512) == 16 and group(2048) == 16 and group(2049) == 32 and group(2048, 2048) == 16
    assert group(2048, 4096) == 32 and group(2047, 32768) == 32 and group(1024, 8192) == 32 and group(1024, 2048) == 16
    assert group(1023, 32768) == 16 and group(512, 8192) == 16


def test_shapes_of_the_kernel_for_17_to_64_rows():
    """Workgroup shape and K splits for the layer shapes it was measured on: wide matrices are not divided
    (six waves), narrow ones are divided until every compute unit has a workgroup, short walks take the
    smaller workgroup and long ones the larger."""
    from llm_runtime_study_amd.kernels import ops

    units = ops.compute_units()
    if units not in (0, 256):
        return
    assert ops.gemm_mid_shape(24576, 4096) == (6, 1) and ops.gemm_mid_shape(151936, 4096) == (6, 1)
    assert ops.gemm_mid_shape(6144, 4096) == (6, 4)
    assert ops.gemm_mid_shape(4096, 4096) == (4, 4) and ops.gemm_mid_shape(4096, 12288) == (8, 8)
    # 34,816 rows (the 14B feed-forward): 363 workgroups of six waves or 544 of four leave the chip's last round half empty, 436 of five do not
    assert ops.gemm_mid_shape(34816, 5120) == (5, 1) and ops.gemm_mid_shape(24576, 4096) == (6, 1) and ops.gemm_mid_shape(151936, 4096)[0] == 6
    # 51,200 rows (the 32B feed-forward): 400 workgroups of eight waves, two rounds, fetch least for the busiest unit
    assert ops.gemm_mid_shape(51200, 5120) == (8, 1)
    # the deal of the rows for a given number of rows of the product: the 14B feed-forward evenly, 256 workgroups of 8
    # tiles of which 128 have a ninth; the 32B one 512 of 6, 128 with a seventh; the LM head 1,536 of 6, 280 with a
    # seventh; those whose rows divide evenly as their shapes say
    for m in (17, 40, 64):
        assert ops.gemm_mid_deal(m, 34816, 5120) == (8, 1, 256, 128) and ops.gemm_mid_deal(m, 51200, 5120) == (6, 1, 512, 128)
        assert ops.gemm_mid_deal(m, 24576, 4096) == (6, 1, 256, 0) and ops.gemm_mid_deal(m, 4096, 4096) == (4, 4, 64, 0)
    assert ops.gemm_mid_deal(64, 151936, 4096) == (6, 1, 1536, 280)
    assert ops.gemm_mid_deal(64, 51200, 5120, ops.KernelChoice(mid_even=1)) == (8, 1, 400, 0)
    assert ops.gemm_mid_deal(100, 34816, 5120)[3] == 0            # beyond 64 rows the plain deal only
    assert ops.gemm_mid_deal(64, 34816, 5120, ops.KernelChoice(mid_even=1)) == (5, 1, 436, 0)
    for n, k in ((64, 256), (208, 512), (5120, 5120), (5120, 17408), (7168, 5120), (51200, 5120), (1040, 3328)):
        waves, splits = ops.gemm_mid_shape(n, k)
        assert waves in (4, 5, 6, 8) and 1 <= splits <= 8 and (splits == 1 or k // 256 // splits >= 2)


def test_the_route_of_a_product_follows_rows_dtype_and_the_runners_choices():
    """`plan()` of parts/linear.py: one decision per class of (rows, shape, dtype, form of the input), and the
    choices a runner carries move it; nothing in the process does."""
    import torch

    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.kernels.ops import KernelChoice
    from llm_runtime_study_amd.parts.linear import ROUTES, plan

    bf16, f32 = torch.bfloat16, torch.float32

    def route(m, n, k, arrives="tensor", dtype=bf16, out=bf16, **more):
        got = plan(m, n, k, weight_dtype=dtype, run_dtype=dtype, out_dtype=out, arrives=arrives, **more)
        assert got[0] in ROUTES
        return got

    # decode, at most 16 rows: the norm arrives begun and the next one is begun (o_proj, down), or only finished (qkv, gate_up)
    assert route(8, 4096, 4096, "scaled", out=f32, accumulate=True, norm_follows=4096) == ("chain", "")
    assert route(8, 24576, 4096, "scaled", swiglu=True) == ("chain", "")
    assert route(8, 4096, 4096, out=f32, accumulate=True, norm_follows=4096) == ("chain", "")     # a plain input, the next norm begun
    assert route(8, 4096, 4096, out=f32, accumulate=True) == ("own", "")                          # nothing to fold in: the few-rows kernel by shape
    # the first product of a step: the residual stream, normalised on the way in where that pays (narrow matrices)
    assert route(8, 4096, 4096, "lazy") == ("fused_norm", "")
    assert route(8, 24576, 4096, "lazy", swiglu=True) == ("own", "materialize")
    assert route(1, 151936, 4096, "lazy", out=f32) == ("own", "materialize")
    # 17..128 rows
    assert route(64, 6144, 4096, "scaled") == ("mid_scaled", "")
    assert route(64, 4096, 12288, out=f32, accumulate=True, norm_follows=4096) == ("mid_begin", "")
    assert route(64, 4096, 12288, out=f32, accumulate=True, norm_follows=4096, out_contiguous=False) == ("mid", "")
    assert route(128, 24576, 4096, swiglu=True) == ("mid", "")
    assert route(64, 4096, 4000) == ("library", "")                                               # K no multiple of 256: not that kernel's
    assert route(64, 4096, 4000, choice=KernelChoice(library=False)) == ("own", "")
    assert route(64, 6144, 4096, "scaled", choice=KernelChoice(mid=False)) == ("library", "materialize")
    assert route(64, 6144, 4096, "scaled", choice=KernelChoice(mid=False, library=False)) == ("own", "materialize")
    assert route(64, 6144, 4096, "lazy", choice=KernelChoice(few_rows_max=64)) == ("mid", "materialize")   # 6,144 rows: folding the norm in does not pay
    assert route(64, 4096, 4096, "lazy", choice=KernelChoice(few_rows_max=64)) == ("fused_norm", "")
    # many rows
    assert route(2048, 24576, 4096, swiglu=True) == ("library", "")
    assert route(2048, 4096, 4096, out=f32, accumulate=True, norm_follows=4096) == ("library", "")
    assert route(2048, 4096, 4096, bias=True) == ("own", "")
    assert route(2048, 4096, 4096, contiguous=False) == ("own", "")
    assert route(2048, 24576, 4096, swiglu=True, choice=KernelChoice(library=False)) == ("own", "")
    assert route(129, 4096, 4096) == ("library", "") and route(128, 4096, 4096) == ("mid", "")
    # a prompt portion of a few hundred rows: too few tiles for the chip; with a long K (or up to 256 rows) this
    # package's kernel with K divided between workgroups, else the library
    if ops.compute_units() in (0, 256):
        # ... whose finishing kernel also adds the residual and normalises the rows when an RMSNorm follows
        assert route(512, 5120, 17408, out=f32, accumulate=True, norm_follows=5120) == ("split_norm", "")
        assert route(512, 4096, 12288, out=f32, accumulate=True, norm_follows=4096) == ("split_norm", "")
        assert route(512, 4096, 12288, out=f32, accumulate=True) == ("own", "")
        assert route(256, 7168, 5120) == ("own", "") and route(512, 7168, 5120) == ("library", "")
        assert route(512, 4096, 4096, out=f32, accumulate=True, norm_follows=4096) == ("library", "")
        assert route(512, 34816, 5120, swiglu=True) == ("library", "")
        assert route(512, 4096, 12288, out=f32, accumulate=True, out_contiguous=False) == ("library", "")
    # float32 runs: this package's own kernels whatever the rows
    for m in (1, 8, 64, 2048):
        assert route(m, 4096, 4096, dtype=f32, out=f32) == ("own", "")
        assert route(m, 4096, 4096, "lazy", dtype=f32, out=f32) == ("own", "materialize")


def test_kernel_choices_travel_with_the_call():
    from llm_runtime_study_amd.errors import KernelError
    from llm_runtime_study_amd.kernels import ops
    import pytest

    assert ops.DEFAULT_CHOICE.word == 3 and ops.KernelChoice(mid=False, whole_lines=False).word == 0
    assert ops.KernelChoice(mid_waves=6, mid_splits=4).word == 3 | 6 << 4 | 4 << 8
    for bad in (dict(few_rows_max=0), dict(few_rows_max=65), dict(mid_waves=7), dict(mid_splits=17)):
        with pytest.raises(KernelError):
            ops.KernelChoice(**bad)
    assert not hasattr(ops, "gemm_mid_tune") and not hasattr(ops, "set_skinny_max_m") and not hasattr(ops, "gemm_skinny_lines")
    if ops.compute_units() in (0, 256):
        assert ops.gemm_mid_shape(4096, 4096, ops.KernelChoice(mid_waves=8, mid_splits=2)) == (8, 2)
        assert ops.gemm_mid_shape(4096, 4096) == (4, 4)


def test_the_generated_plan_dispatch_is_in_step_with_the_entry_point_table():
    """csrc/plan_dispatch.inc is made from ops.PLAN_OPS and ops._SIGNATURES; whoever changes an entry point's
    arguments has to make it again (python -m llm_runtime_study_amd.kernels.plan_codegen)."""
    from llm_runtime_study_amd.kernels import ops, plan_codegen

    assert plan_codegen.TARGET.read_text() == plan_codegen.generate()
    assert len(set(ops.PLAN_OPS)) == len(ops.PLAN_OPS) and all(ops._SIGNATURES[name][1][-1] is not None for name in ops.PLAN_OPS)


def test_a_plan_packs_one_word_per_argument():
    from llm_runtime_study_amd.kernels import ops

    plan = ops.Plan([("lrs_add_into", (0x7F0000001000, 0x7F0000002000, 1, 1 << 33)),
                     ("lrs_scale_rows", (1, 2, 3, 4, 5, 6, 0.5)), ("lrs_fill_i32", (None, -7, 12))])
    words = list(plan.words)[:plan.length]
    assert plan.launches == 3 and plan.length == 5 + 8 + 4
    assert words[:5] == [ops.PLAN_OPS.index("lrs_add_into"), 0x7F0000001000, 0x7F0000002000, 1, 1 << 33]
    assert words[5] == ops.PLAN_OPS.index("lrs_scale_rows") and words[12] == 0x3F000000        # 0.5 as its 32 bits
    assert words[13:] == [ops.PLAN_OPS.index("lrs_fill_i32"), 0, (1 << 64) - 7, 12]               # None: a null pointer; -7: two's complement


def test_the_tile_width_of_the_many_rows_kernel_follows_the_rounds_of_the_chip():
    """`lrs_gemm_lines_width`: K a multiple of 64 and a 256 x 128 tile for every compute unit, then the width
    that needs the fewest rounds times its width (the shapes of the 8B layer at 2,048 rows: one round each)."""
    from llm_runtime_study_amd.kernels import ops

    if ops.compute_units() not in (0, 256):
        return
    assert ops.gemm_lines_width(2048, 24576, 4096) == 256      # 768 tiles: three rounds
    assert ops.gemm_lines_width(2048, 6144, 4096) == 192       # 256 tiles of 192: one round
    assert ops.gemm_lines_width(2048, 4096, 12288) == 128      # 256 tiles of 128
    assert ops.gemm_lines_width(8192, 4096, 4096) == 256       # 512 tiles: two rounds of 256 tie with four of 128
    assert ops.gemm_lines_width(1024, 4096, 4096) == 0         # not a tile for every compute unit
    assert ops.gemm_lines_width(2048, 4096, 4000) == 0         # K no multiple of 64
    assert ops.gemm_lines_width(129, 151936, 4096) == 128      # the LM head of a small step: five rounds of 128 against three of 256
    # too few tiles for the chip: K in as many parts as fill it in one round, each with 8 slices of 64 or more
    assert ops.gemm_lines_splits(512, 4096, 4096) == 4         # 64 tiles x 4
    assert ops.gemm_lines_splits(512, 5120, 17408) == 3        # 80 tiles x 3 = 240
    assert ops.gemm_lines_splits(512, 7168, 5120) == 2         # 112 tiles x 2
    assert ops.gemm_lines_splits(300, 9000, 1088) == 1         # 142 tiles, more than half the units: as they are
    assert ops.gemm_lines_splits(512, 4096, 512) == 0          # one part of 8 slices, 64 tiles: under half the units
    assert ops.gemm_lines_splits(2048, 4096, 4096) == 0        # a tile for every unit: not divided
    assert ops.gemm_lines_splits(128, 4096, 4096) == 0         # the kernel for 17..128 rows' size
    # ... and where that form is taken instead of the vendor library: a long K at any such row count, others up to 256 rows
    assert ops.gemm_split_pays(512, 5120, 17408) and ops.gemm_split_pays(1024, 4096, 12288) and ops.gemm_split_pays(300, 4096, 12288)
    assert ops.gemm_split_pays(256, 5120, 5120) and not ops.gemm_split_pays(512, 5120, 5120)
    assert not ops.gemm_split_pays(256, 4096, 4096)            # 8 parts of 8 slices: too short
    assert not ops.gemm_split_pays(2048, 4096, 12288) and not ops.gemm_split_pays(512, 34816, 5120)


def test_a_recording_of_launches_belongs_to_its_thread():
    """Two runners stepping on two threads each write their own launches down: a recording that is open on one
    thread is not seen, and cannot be closed, from another."""
    import threading

    import pytest

    from llm_runtime_study_amd.errors import KernelError
    from llm_runtime_study_amd.kernels import ops

    ops.record_begin()
    try:
        with pytest.raises(KernelError, match="already open"):
            ops.record_begin()
        seen = {}

        def other():
            try:
                ops.record_end()
            except KernelError as exc:
                seen["end"] = str(exc)
            ops.record_begin()                       # its own, beside the first thread's
            seen["plan"] = ops.record_end().launches

        worker = threading.Thread(target=other)
        worker.start()
        worker.join()
        assert "no recording" in seen["end"] and seen["plan"] == 0
        assert ops.record_end().launches == 0        # still open here
    finally:
        ops.record_drop()


def test_changing_a_runners_kernels_or_plans_forgets_what_was_recorded():
    """A recorded plan holds the kernels that were chosen when it was made: changing the choice, or switching plans
    off and on, on a live runner empties what it had recorded."""
    import torch

    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine.step import ModelRunner, RecordedStep
    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.models import DecoderModel
    from tests.helpers import TINY_A

    model = DecoderModel(spec_for(config_from_dict(TINY_A)))
    cache = CacheManager(model.cache_needs(), page_size=16, num_pages=4, max_requests=2, max_seq_len=64, device="cpu", allocate_storage=False)
    runner = ModelRunner(model, cache, max_step_tokens=16, dtype=torch.float32, device="cpu")
    assert runner.use_plans and runner.kernels.library
    runner._plans[("shape",)] = RecordedStep(ops.Plan([]), 0, None)
    runner.kernels = runner.kernels                  # the same choice: nothing to forget
    assert len(runner._plans) == 1
    runner.kernels = ops.KernelChoice(library=False)
    assert not runner._plans and not runner.library_gemm
    runner._plans[("shape",)] = RecordedStep(ops.Plan([]), 0, None)
    runner.use_plans = False
    assert not runner._plans and not runner.use_plans
