"""The token choice that allocates nothing (lrs_choose_tokens_static), called through ctypes, against the
existing two-pass entry point (lrs_choose_tokens_split) that takes its scratch as arguments."""

import ctypes
from ctypes import c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from llm_runtime_study_amd.kernels import ops

    lib = ctypes.CDLL(ops.loaded_library_path())
    lib.lrs_last_error.restype = ctypes.c_char_p
    lib.lrs_choose_tokens_static.restype = c_int
    lib.lrs_choose_tokens_static.argtypes = [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
    lib.lrs_choose_tokens_split.restype = c_int
    lib.lrs_choose_tokens_split.argtypes = [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
    lib.lrs_choose_tokens_static_max_parts.restype = c_int
    lib.lrs_choose_tokens_static_init.restype = c_int
    return lib


def _case(rows, vocab, seed, sampled):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, vocab, generator=gen).cuda()
    logits[0, vocab - 1] = 50.0            # a winner in the last slice
    if rows > 1:
        logits[1, 7] = logits[1, vocab // 2] = 40.0   # a tie between slices: the lower index wins
    temperature = seeds = counters = None
    if sampled:
        temperature = torch.linspace(0.0, 1.5, rows).cuda()
        seeds = torch.arange(rows, dtype=torch.int64).cuda() * 7919 + seed
        counters = (torch.arange(rows, dtype=torch.int32) % 5).cuda()
    return logits, temperature, seeds, counters


def _pointer(t):
    return None if t is None else t.data_ptr()


@pytest.mark.parametrize("sampled", [False, True])
def test_static_choice_equals_the_split_entry_point_on_two_calls_in_a_row(sampled):
    lib = _library()
    assert lib.lrs_choose_tokens_static_init() == 0, lib.lrs_last_error().decode()
    stream = torch.cuda.current_stream().cuda_stream
    # the second call is smaller in rows, vocabulary and slices: whatever the first left in the scratch must not show
    for rows, vocab, parts, seed in ((24, 151936, 38, 1), (5, 33331, 9, 2)):
        logits, temperature, seeds, counters = _case(rows, vocab, seed, sampled)
        expected = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        part_value = torch.empty(rows * parts, dtype=torch.float32, device="cuda")
        part_index = torch.empty(rows * parts, dtype=torch.int32, device="cuda")
        rc = lib.lrs_choose_tokens_split(expected.data_ptr(), logits.data_ptr(), logits.stride(0), rows, vocab, _pointer(temperature),
                                         _pointer(seeds), _pointer(counters), part_value.data_ptr(), part_index.data_ptr(), parts, 0, stream)
        assert rc == 0, lib.lrs_last_error().decode()
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        # free device memory as the driver sees it: an allocation inside the library (not only one of torch's) would show
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = lib.lrs_choose_tokens_static(got.data_ptr(), logits.data_ptr(), logits.stride(0), rows, vocab, _pointer(temperature),
                                          _pointer(seeds), _pointer(counters), parts, 0, stream)
        assert rc == 0, lib.lrs_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
        assert got.tolist() == expected.tolist()
        if not sampled:
            assert got.tolist() == logits.argmax(dim=1).tolist()
            assert got[0].item() == vocab - 1 and (rows == 1 or got[1].item() == 7)


def test_static_choice_refuses_more_slices_than_its_scratch_holds():
    lib = _library()
    most = lib.lrs_choose_tokens_static_max_parts()
    rows, parts = 64, most // 64 + 1
    logits = torch.zeros(rows, 1024, device="cuda")
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    rc = lib.lrs_choose_tokens_static(out.data_ptr(), logits.data_ptr(), logits.stride(0), rows, 1024, None, None, None, parts, 0,
                                      torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and "more than" in lib.lrs_last_error().decode()
    torch.cuda.synchronize()


def test_static_choice_can_be_captured_in_a_graph():
    """Under stream capture an allocation is an error, so a call that is captured and whose replays give the
    tokens of the eager call has allocated nothing."""
    from llm_runtime_study_amd.kernels import ops

    lib = _library()
    assert lib.lrs_choose_tokens_static_init() == 0, lib.lrs_last_error().decode()
    rows, vocab, parts = 6, 50021, 13
    logits, *_ = _case(rows, vocab, 3, False)
    got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.graph_begin()
        try:
            rc = lib.lrs_choose_tokens_static(got.data_ptr(), logits.data_ptr(), logits.stride(0), rows, vocab, None, None, None, parts, 0,
                                              side.cuda_stream)
        finally:
            graph = ops.graph_end()
        assert rc == 0, lib.lrs_last_error().decode()
        try:
            for turn in range(3):
                logits[turn, 11 + turn] = 90.0          # another winner every replay
                got.fill_(-1)
                ops.graph_launch(graph)
                side.synchronize()
                assert got.tolist() == logits.argmax(dim=1).tolist()
        finally:
            ops.graph_destroy(graph)


def test_static_choice_refuses_rows_that_are_not_finite():
    lib = _library()
    rows, vocab, parts = 4, 20000, 5
    logits, *_ = _case(rows, vocab, 4, False)
    logits[1, 19999] = float("nan")
    logits[3, 5] = float("-inf")
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.lrs_choose_tokens_static(out.data_ptr(), logits.data_ptr(), logits.stride(0), rows, vocab, None, None, None, parts, 0, stream)
    assert rc == 0, lib.lrs_last_error().decode()
    torch.cuda.synchronize()
    assert out.tolist() == [vocab - 1, -1, int(logits[2].argmax()), -1]
