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
    for workgroups in (1, 8, 24, 64, 200):
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
    assert splits(8, 2048, 1 << 16) == 2                # at least 1,024 keys each
    assert splits(8, 1 << 20, 16 << 20) == 4            # partial results stay within 256 MB


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
    for n, k in ((64, 256), (208, 512), (5120, 5120), (5120, 17408), (7168, 5120), (51200, 5120), (1040, 3328)):
        waves, splits = ops.gemm_mid_shape(n, k)
        assert waves in (4, 6, 8) and 1 <= splits <= 8 and (splits == 1 or k // 256 // splits >= 2)
