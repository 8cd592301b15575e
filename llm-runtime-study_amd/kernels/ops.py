"""Python face of the gfx950 kernel library.

Every function checks on the host that the operand shapes, dtypes and strides are what
its kernel assumes, then launches on the current torch stream.  Nothing here computes
with torch: tensors are only containers of device memory.  Loading fails loudly when
the library is missing or cannot be built; there is no fallback.
"""

from __future__ import annotations

import functools
import threading

from dataclasses import dataclass
import ctypes
import struct
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p, POINTER, byref

import torch

from ..errors import KernelError
from . import build as _build

_lib = None
_lib_path = ""

F32, BF16 = 0, 1
OUT_STORE, OUT_STORE_F32, OUT_ADD_F32 = 0, 1, 2


@dataclass(frozen=True)
class KernelChoice:
    """Which matrix-product kernels a caller wants where there is a choice.  A step carries its runner's
    (`ctx.kernels`); measurements and tests make their own.  Nothing of it is kept in the kernel library:
    the parts that concern a kernel travel with every call.

    few_rows_max   rows up to which the few-rows kernels (and the norms folded into them) are used: 16 in
                   steps, since from 17 rows on other kernels are faster; the kernels themselves take 64
    mid            the kernel for 17..128 rows may be used
    mid_waves, mid_splits   its workgroup shape (4, 5, 6 or 8 waves) and number of K splits (0: its own choice)
    mid_even       its weight rows dealt out evenly over a whole multiple of the compute units, some workgroups with
                   16 rows more than the others: 0 where it pays (its own choice), 1 never, 2 wherever the shape allows
    whole_lines    the few-rows kernel loads its weights as whole 128-byte lines where the shape allows
    library        bfloat16 products of more rows than these kernels are made for go to the vendor's matrix
                   library (as the reference leaves them to nn.Linear); else to this package's own kernel"""

    few_rows_max: int = 16
    mid: bool = True
    mid_waves: int = 0
    mid_splits: int = 0
    mid_even: int = 0
    whole_lines: bool = True
    library: bool = True

    def __post_init__(self):
        if not 1 <= self.few_rows_max <= 64:
            raise KernelError(f"the few-rows kernel takes 1..64 rows, got few_rows_max={self.few_rows_max}")
        if self.mid_waves not in (0, 4, 5, 6, 8) or not 0 <= self.mid_splits <= 16:
            raise KernelError(f"the kernel for 17..128 rows has 4, 5, 6 or 8 waves and 1..16 K splits (0: its own choice), got {self.mid_waves} and {self.mid_splits}")
        if self.mid_even not in (0, 1, 2):
            raise KernelError(f"mid_even is 0 (where it pays), 1 (never) or 2 (wherever the shape allows), got {self.mid_even}")

    @property
    def word(self) -> int:
        """The choices a kernel launch needs, as the one integer the entry points take."""
        return int(self.mid) | int(self.whole_lines) << 1 | self.mid_waves << 4 | self.mid_splits << 8 | self.mid_even << 13


DEFAULT_CHOICE = KernelChoice()

_SIGNATURES = {
    "lrs_last_error": (c_char_p, []),
    "lrs_plan_run": (c_int, [c_void_p, c_int64, c_int, c_void_p]),
    "lrs_device_arch": (c_int, [c_int, c_char_p, c_int, POINTER(c_int)]),
    "lrs_graph_begin": (c_int, [c_void_p]),
    "lrs_graph_end": (c_int, [c_void_p, POINTER(c_void_p)]),
    "lrs_graph_launch": (c_int, [c_void_p, c_void_p]),
    "lrs_graph_destroy": (c_int, [c_void_p]),
    "lrs_copy_h2d": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "lrs_copy_h2d_scatter": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "lrs_embed": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_rmsnorm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_add_rmsnorm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_rope_table": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_qk_prep": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float,
                            c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm_mid_qk_prep": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_float, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p, c_int64, c_void_p]),
    "lrs_silu_mul": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_add_into": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_void_p]),
    "lrs_fill_i32": (c_int, [c_void_p, c_int, c_int64, c_void_p]),
    "lrs_step_prepare": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "lrs_step_prepare_summary_size": (c_int, []),
    "lrs_scatter_i32": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_gather_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                         c_int, c_float, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "lrs_gemm_workspace_bytes": (c_int64, []),
    "lrs_gemm_lines_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p, c_int,
                                           c_void_p, c_int64, c_void_p]),
    "lrs_gemm_norm_chain": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm_norm_chain_parts": (c_int, [c_int]),
    "lrs_scale_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_gemm_skinny_capacity": (c_int, []),
    "lrs_advance_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_advance_slots": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]),
    "lrs_copy_to_pinned": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "lrs_stream_read": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_void_p]),
    "lrs_probe_lds": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p]),
    "lrs_probe_mfma": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_probe_lines": (c_int, [c_void_p, c_size_t, c_void_p, c_int, c_int, c_size_t, c_int, c_void_p]),
    "lrs_gemm_prepare": (c_int, []),
    "lrs_library_gemm_prepare": (c_int, []),
    "lrs_library_gemm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_host_device_pointer": (c_int, [c_void_p, POINTER(c_void_p)]),
    "lrs_gemm_mid_shape": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p]),
    "lrs_gemm_mid_deal": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lrs_gemm_mid_scaled": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float, c_int,
                                    c_void_p, c_int64, c_void_p]),
    "lrs_gemm_mid_add_norm_begin": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                            c_void_p, c_int64, c_void_p]),
    "lrs_norm_begin_parts": (c_int, [c_int]),
    "lrs_attention": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "lrs_attention_decode": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_attention_prefill": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                      c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p]),
    "lrs_attention_prefill_prepares": (c_int, [c_int]),
    "lrs_compute_units": (c_int, []),
    "lrs_gemm_lines_width": (c_int, [c_int, c_int, c_int]),
    "lrs_gemm_lines_splits": (c_int, [c_int, c_int, c_int]),
    "lrs_gemm_lines_split_pays": (c_int, [c_int, c_int, c_int]),
    "lrs_attention_prefill_group": (c_int, []),
    "lrs_attention_prefill_group_for": (c_int, [c_int, c_int]),
    "lrs_choose_tokens": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_choose_tokens_split": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_choose_tokens_static": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_choose_tokens_static_init": (c_int, []),
    "lrs_choose_tokens_static_max_parts": (c_int, []),
    "lrs_filter_logits": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
}


def library():
    """Load (building first if needed) the kernel library; raises KernelError if impossible."""
    global _lib, _lib_path
    if _lib is None:
        try:
            path = _build.ensure_built()
            lib = ctypes.CDLL(str(path))
            _lib_path = str(path)
        except (_build.BuildError, OSError) as exc:
            raise KernelError(f"the HIP kernel library is not available: {exc}") from exc
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
        if torch.cuda.is_available():
            torch.cuda.init()
            _check(lib.lrs_gemm_prepare())   # device scratch is made now, never inside a step
            _check(lib.lrs_choose_tokens_static_init())
            _check(lib.lrs_library_gemm_prepare())
    return _lib


# ------------------------------------------------------------ launch plans
# Every kernel launch goes through _launch().  While a recording is open, the launch (entry point and
# arguments, without the stream) is also written down; the recording becomes a Plan, an array of 64-bit words
# that lrs_plan_run() walks in one call, making the same launches with the same arguments on the stream it
# is given.  A step whose shape has been seen before is then one call into the library instead of some
# hundreds of Python calls.  What is written down are addresses and sizes: a plan is good for as long as
# every buffer it names lives where it lived (the caller's business: see engine/step.py).
#
# PLAN_OPS fixes the number of each entry point inside a plan; csrc/plan_dispatch.inc, made from this list
# and _SIGNATURES by kernels/plan_codegen.py, is the other side (a test keeps the two in step).
PLAN_OPS = ("lrs_add_into", "lrs_add_rmsnorm", "lrs_advance_decode", "lrs_advance_slots", "lrs_attention", "lrs_attention_decode",
            "lrs_attention_prefill", "lrs_choose_tokens", "lrs_choose_tokens_split", "lrs_copy_to_pinned", "lrs_embed", "lrs_fill_i32",
            "lrs_filter_logits", "lrs_gather_rows", "lrs_gemm", "lrs_gemm_lines_add_rmsnorm", "lrs_gemm_mid_add_norm_begin", "lrs_gemm_mid_qk_prep", "lrs_gemm_mid_scaled",
            "lrs_gemm_norm_chain", "lrs_library_gemm", "lrs_qk_prep", "lrs_rmsnorm", "lrs_rope_table", "lrs_scale_rows", "lrs_silu_mul")
_PLAN_INDEX = {name: index for index, name in enumerate(PLAN_OPS)}


class _Recording(threading.local):
    """The recording that is open on this thread, if any: launches made on another thread (a second runner, a
    sampler) are none of its business."""
    calls: list | None = None


_recording = _Recording()


class Plan:
    """A recorded sequence of launches, ready for plan_run()."""

    def __init__(self, calls: list):
        words: list[int] = []
        for name, args in calls:
            argtypes = _SIGNATURES[name][1][:-1]
            words.append(_PLAN_INDEX[name])
            for kind, value in zip(argtypes, args):
                if kind is c_float:
                    words.append(int.from_bytes(struct.pack("<f", value), "little"))
                elif value is None:
                    words.append(0)
                else:
                    words.append(int(value) & 0xFFFFFFFFFFFFFFFF)
        self.launches = len(calls)
        self.words = (ctypes.c_uint64 * max(len(words), 1))(*words)
        self.length = len(words)


def record_begin() -> None:
    """Start writing down the launches this thread makes (they still run as they are made)."""
    if _recording.calls is not None:
        raise KernelError("a recording of launches is already open")
    _recording.calls = []


def record_end() -> Plan:
    """Stop writing launches down; returns the plan of those made since record_begin()."""
    if _recording.calls is None:
        raise KernelError("no recording of launches is open")
    calls, _recording.calls = _recording.calls, None
    return Plan(calls)


def record_drop() -> None:
    """Stop writing launches down and forget them (after a failure)."""
    _recording.calls = None


def plan_run(plan: Plan) -> None:
    """Make the plan's launches, in order, on the current stream."""
    if plan.launches:
        _check(library().lrs_plan_run(plan.words, plan.length, plan.launches, _stream()))


def _launch(name: str, *args) -> None:
    code = getattr(_lib or library(), name)(*args)
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())
    if _recording.calls is not None:
        if name not in _PLAN_INDEX:
            raise KernelError(f"{name} cannot be part of a recorded plan")
        _recording.calls.append((name, args[:-1]))


def loaded_library_path() -> str:
    library()
    return _lib_path


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())


# The handle of the current stream is asked for at every kernel launch; the raw query costs a
# fraction of a microsecond where torch.cuda.current_stream() builds an object in about nine.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, got {dtype}")


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(t: torch.Tensor, name: str, dtype=None) -> int:
    _need(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a device tensor")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must be {dtype}, got {t.dtype}")
    return t.data_ptr()


def pinned_device_address(t: torch.Tensor) -> int:
    """The address under which kernels see the pinned host tensor `t`.  The owner of the tensor asks
    once and keeps the answer with the tensor (asking whether memory is pinned is slow)."""
    _need(not t.is_cuda and t.is_contiguous() and t.is_pinned(), "pinned_device_address needs a contiguous pinned host tensor")
    out = c_void_p()
    _check(library().lrs_host_device_pointer(t.data_ptr(), byref(out)))
    return out.value


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be 2-D with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def device_arch(device: int = 0) -> tuple[str, int]:
    buf = ctypes.create_string_buffer(256)
    cus = c_int(0)
    _check(library().lrs_device_arch(device, buf, 256, byref(cus)))
    return buf.value.decode(), cus.value


# ----------------------------------------------------------------- graphs
def graph_begin() -> None:
    _check(library().lrs_graph_begin(_stream()))


def graph_end() -> int:
    handle = c_void_p()
    _check(library().lrs_graph_end(_stream(), byref(handle)))
    return handle.value


def graph_launch(handle: int) -> None:
    _check(library().lrs_graph_launch(handle, _stream()))


def graph_destroy(handle: int) -> None:
    library().lrs_graph_destroy(handle)


def copy_h2d(dst: torch.Tensor, src: torch.Tensor, count: int) -> None:
    """Asynchronous copy of the first `count` elements of `src` into device `dst`.  `src` must be
    pinned host memory (the caller checks that once, when it allocates it: asking is slow)."""
    _need(src.device.type == "cpu" and src.is_contiguous() and dst.is_contiguous(), "copy_h2d needs a contiguous host source and a contiguous destination")
    _need(src.dtype == dst.dtype and 0 < count <= src.numel() and count <= dst.numel(), "copy_h2d: size or dtype mismatch")
    _launch("lrs_copy_h2d", _dev(dst, "dst"), src.data_ptr(), count * src.element_size(), _stream())


def copy_h2d_scatter(dst: torch.Tensor, src: torch.Tensor, count: int, tables: torch.Tensor, pairs_at: int, pairs: int) -> None:
    """copy_h2d() of the first `count` int32 elements (a multiple of 4) of pinned `src`, and in the same launch the `pairs`
    (offset, value) pairs that lie in `src` from element `pairs_at` (even) on written into `tables` (int32, on the
    device): tables.view(-1)[offset] = value.  The caller has checked the offsets."""
    _need(src.device.type == "cpu" and src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype == torch.int32,
          "copy_h2d_scatter needs contiguous int32 tensors, the source on the host")
    _need(0 <= count <= src.numel() and count <= dst.numel() and count % 4 == 0, "copy_h2d_scatter: the count must be a multiple of 4 inside both tensors (0: only the pairs)")
    _need(tables.dtype == torch.int32 and tables.is_contiguous() and pairs > 0 and pairs_at % 2 == 0 and pairs_at + 2 * pairs <= src.numel(),
          "copy_h2d_scatter: int32 tables and pairs inside the source, from an even element on")
    _launch("lrs_copy_h2d_scatter", _dev(dst, "dst"), src.data_ptr(), count * 4, _dev(tables, "tables"), pairs_at * 4, pairs, _stream())


def stream_read(src: torch.Tensor, sink: torch.Tensor, blocks: int) -> None:
    """Reads all of `src` once with `blocks` workgroups (a probe of the memory rate a kernel can reach)."""
    _need(src.is_contiguous() and sink.dtype == torch.int32 and sink.numel() >= blocks, "stream_read: contiguous source and an int32 sink of `blocks` elements")
    _launch("lrs_stream_read", _dev(src, "src"), src.numel() * src.element_size(), _dev(sink, "sink"), blocks, _stream())



def probe_lds(sink: torch.Tensor, blocks: int, iters: int, stride: int) -> None:
    """`blocks` workgroups read LDS `iters` x 8 times, 16 bytes a lane, rows `stride` bytes apart (microbench lds)."""
    _need(sink.dtype == torch.int32 and sink.numel() >= 256, "probe_lds: an int32 sink of 256 elements")
    _launch("lrs_probe_lds", _dev(sink, "sink"), blocks, iters, stride, _stream())


def probe_lines(data: torch.Tensor, sink: torch.Tensor, blocks: int, threads: int, bytes_each: int, pattern: int) -> None:
    """Measurement only: `blocks` workgroups stream `bytes_each` bytes each of `data` with 16-byte loads in the lane
    order `pattern` (0 fragment order, 1 whole lines, 2 a row to four neighbouring lanes)."""
    _need(sink.dtype == torch.int32 and sink.numel() >= 256, "probe_lines: an int32 sink of 256 elements")
    _need(data.is_contiguous(), "probe_lines: data must be contiguous")
    _launch("lrs_probe_lines", _dev(data, "data"), data.numel() * data.element_size(), _dev(sink, "sink"), blocks, threads, bytes_each, pattern, _stream())


def probe_mfma(sink: torch.Tensor, blocks: int, iters: int, valu: int, exps: bool) -> None:
    """`blocks` workgroups issue `iters` x 32 matrix instructions with `valu` multiply-adds after each (microbench mfma)."""
    _need(sink.dtype == torch.float32 and sink.numel() >= 256, "probe_mfma: a float32 sink of 256 elements")
    _launch("lrs_probe_mfma", _dev(sink, "sink"), blocks, iters, valu, int(bool(exps)), _stream())

def copy_to_pinned(dst: torch.Tensor, src: torch.Tensor, count: int) -> None:
    """The first `count` elements of device `src` into pinned host `dst`, by a kernel (the host reads
    them after synchronising the stream).  count * element size must be a multiple of 16."""
    _need(dst.device.type == "cpu" and dst.is_contiguous() and src.is_contiguous(), "copy_to_pinned needs a contiguous pinned host destination and a contiguous source")
    _need(src.dtype == dst.dtype and 0 < count <= src.numel() and count <= dst.numel(), "copy_to_pinned: size or dtype mismatch")
    _launch("lrs_copy_to_pinned", dst.data_ptr(), _dev(src, "src"), count * src.element_size(), _stream())


# ------------------------------------------------------------ elementwise
def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, multiplier: float = 1.0) -> None:
    tokens, hidden = out.shape
    _need(out.is_contiguous() and table.is_contiguous() and table.dim() == 2 and table.shape[1] == hidden, "embed: out [T,H] and table [V,H] must agree")
    _need(ids.dtype == torch.int32 and ids.numel() >= tokens and ids.is_contiguous(), "embed: ids must be int32 [T]")
    _launch("lrs_embed", _dev(out, "out", torch.float32), _dev(table, "table"), dtype_code(table.dtype),
                               _dev(ids, "ids"), tokens, hidden, multiplier, _stream())


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None) -> None:
    n_rows, hidden = out.shape
    _need(out.is_contiguous() and x.is_contiguous() and x.dim() == 2 and x.shape[1] == hidden, "rmsnorm: out and x must be contiguous [*, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"rmsnorm: weight must hold {hidden} values")
    if rows is None:
        _need(x.shape[0] >= n_rows, "rmsnorm: x has fewer rows than out")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows and rows.is_contiguous(), "rmsnorm: rows must be int32")
    _launch("lrs_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x", torch.float32), _dev(weight, "weight"),
                                 dtype_code(weight.dtype), None if rows is None else _dev(rows, "rows"), n_rows, hidden, eps, _stream())


def add_rmsnorm(out: torch.Tensor, x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """x += y (float32 residual stream, bf16 addend), then out = RMSNorm(x) with `weight`, in one pass."""
    n_rows, hidden = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.dtype == torch.bfloat16 and y.is_contiguous() and y.shape == x.shape,
          "add_rmsnorm: x must be contiguous float32 [T, H] and y bf16 of the same shape")
    _need(out.is_contiguous() and out.shape == x.shape, "add_rmsnorm: out must be contiguous [T, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"add_rmsnorm: weight must hold {hidden} values")
    _launch("lrs_add_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"), _dev(y, "y"), _dev(weight, "weight"),
                                     dtype_code(weight.dtype), n_rows, hidden, eps, _stream())


def rope_table(cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> None:
    tokens, half = cos.shape
    _need(cos.is_contiguous() and sin.is_contiguous() and sin.shape == cos.shape, "rope_table: cos and sin must be contiguous [T, half]")
    _need(inv_freq.numel() == half and inv_freq.is_contiguous(), "rope_table: inv_freq must hold `half` values")
    _need(positions.dtype == torch.int32 and positions.numel() >= tokens and positions.is_contiguous(), "rope_table: positions must be int32 [T]")
    _launch("lrs_rope_table", _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32), _dev(positions, "positions"),
                                    _dev(inv_freq, "inv_freq", torch.float32), tokens, half, _stream())


def qk_prep(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float, cos, sin,
            k_pages, v_pages, slots, page_size: int, skip_q: bool = False) -> None:
    """Normalise and rotate the q and k heads of `qkv` [T, (nq+2*nkv)*d]; q in place, k and v into pages.
    skip_q: the q heads are left as they are (attention_prefill() with `prepare` takes them raw)."""
    tokens = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    _need(qkv.shape[1] == (nq + 2 * nkv) * d, f"qk_prep: qkv width {qkv.shape[1]} is not (nq+2nkv)*d = {(nq + 2 * nkv) * d}")
    rot_half = 0
    if cos is not None:
        rot_half = cos.shape[1]
        _need(cos.shape[0] >= tokens and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous(), "qk_prep: rotary tables must be [T, half]")
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32, "qk_prep: rotary tables must be float32")
    w_dtype = qkv.dtype
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == d and k_weight.numel() == d and q_weight.dtype == k_weight.dtype, "qk_prep: q/k norm weights must both hold head_dim values")
        w_dtype = q_weight.dtype
    if nkv > 0:
        _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, d, page_size),
              f"qk_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {d}, {page_size}]")
        _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "qk_prep: pages must be contiguous and of the activation dtype")
        _need(slots.dtype == torch.int32 and slots.numel() >= tokens and slots.is_contiguous(), "qk_prep: slots must be int32 [T]")
    _launch("lrs_qk_prep", 
        _dev(qkv, "qkv"), dtype_code(qkv.dtype), tokens, stride, nq, nkv, d,
        None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"),
        dtype_code(w_dtype), eps, None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half,
        None if nkv == 0 else _dev(k_pages, "k_pages"), None if nkv == 0 else _dev(v_pages, "v_pages"),
        None if nkv == 0 else _dev(slots, "slots"), page_size, int(bool(skip_q)), _stream())


@functools.lru_cache(maxsize=1)
def gemm_workspace_bytes() -> int:
    """Bytes of device memory a caller brings as `workspace` to the products that divide K between workgroups."""
    return int(library().lrs_gemm_workspace_bytes())


def _workspace(t: torch.Tensor | None, name: str) -> tuple:
    """(address, bytes) of a caller's workspace for the sums of K splits; (None, 0): the one the process keeps, which
    all callers that bring none share (their products must then stay on one stream)."""
    if t is None:
        return None, 0
    if isinstance(t, tuple):            # (address, bytes) that workspace_address() has checked before
        return t
    _need(t.is_cuda and t.is_contiguous() and t.numel() * t.element_size() >= gemm_workspace_bytes(),
          f"{name}: the workspace must be a contiguous device tensor of at least {gemm_workspace_bytes()} bytes")
    return t.data_ptr(), t.numel() * t.element_size()


def workspace_address(t: torch.Tensor) -> tuple:
    """(address, bytes) of a workspace tensor, checked once: callers that make many products a step pass this on as
    `workspace` instead of the tensor."""
    return _workspace(t, "workspace")


def gemm_mid_qk_prep_takes(dtype: torch.dtype, m: int, nq: int, nkv: int, d: int, k: int, rot_half: int,
                           choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm_mid_qk_prep() takes the shape: bf16, 17..128 rows, heads the vector form of qk_prep takes
    (head_dim 16, 32, 64, ... 1024, rotation over the whole head or none), cache written by this layer."""
    per_head = d // 16
    return (gemm_mid_takes(dtype, m, (nq + 2 * nkv) * d, k, MID_ROWS_PREFERRED, choice) and nkv > 0 and d % 16 == 0 and 0 < per_head <= 64
            and per_head & (per_head - 1) == 0 and rot_half in (0, d // 2))


def gemm_mid_qk_prep(qkv: torch.Tensor, a: torch.Tensor, w: torch.Tensor, sumsq: torch.Tensor | None, in_eps: float, nq: int, nkv: int,
                     d: int, q_weight, k_weight, eps: float, cos, sin, k_pages, v_pages, slots, page_size: int,
                     choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """The q/k/v product of 17..128 bf16 rows (a @ w.T; with `sumsq` the input is a norm begun before it, as in
    gemm_mid_scaled) and qk_prep() of its result in two kernels: the one that prepares the heads adds up the sums of
    the product's K splits itself.  q goes into `qkv` [M, (nq+2*nkv)*d], k and v into the pages."""
    m, k = a.shape
    n = (nq + 2 * nkv) * d
    rot_half = 0 if cos is None else cos.shape[1]
    _need(a.dtype == torch.bfloat16 and gemm_mid_qk_prep_takes(w.dtype, m, nq, nkv, d, k, rot_half, choice), "gemm_mid_qk_prep: shape not taken (see gemm_mid_qk_prep_takes)")
    _need(w.shape == (n, k) and w.is_contiguous(), f"gemm_mid_qk_prep: weight must be contiguous [{n}, {k}]")
    _need(qkv.dtype == torch.bfloat16 and qkv.shape == (m, n), f"gemm_mid_qk_prep: qkv must be bf16 [{m}, {n}]")
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous() and in_eps > 0, f"gemm_mid_qk_prep: sumsq must be float32 [parts, {m}] and its eps positive")
    if cos is not None:
        _need(cos.shape[0] >= m and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous() and cos.dtype == torch.float32 and sin.dtype == torch.float32,
              "gemm_mid_qk_prep: rotary tables must be float32 [T, half]")
    w_dtype = torch.bfloat16
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == d and k_weight.numel() == d and q_weight.dtype == k_weight.dtype, "gemm_mid_qk_prep: q/k norm weights must both hold head_dim values")
        w_dtype = q_weight.dtype
    _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, d, page_size),
          f"gemm_mid_qk_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {d}, {page_size}]")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16, "gemm_mid_qk_prep: pages must be contiguous bf16")
    _need(slots.dtype == torch.int32 and slots.numel() >= m and slots.is_contiguous(), "gemm_mid_qk_prep: slots must be int32 [T]")
    _launch("lrs_gemm_mid_qk_prep", 
        _dev(qkv, "qkv"), _rows(qkv, "qkv"), _dev(a, "a"), _dev(w, "w"), m, k, _rows(a, "a"),
        None if sumsq is None else _dev(sumsq, "sumsq"), 0 if sumsq is None else sumsq.shape[0], in_eps if sumsq is not None else 0.0,
        nq, nkv, d, None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"),
        dtype_code(w_dtype), eps, None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half,
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(slots, "slots"), page_size, choice.word,
        *_workspace(workspace, "gemm_mid_qk_prep"), _stream())


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor, interleaved: bool = False) -> None:
    """out = silu(gate) * up; gate_up holds [gate | up], or groups of 8 gate then 8 up columns if `interleaved`."""
    tokens, inter = out.shape
    _need(out.is_contiguous() and gate_up.is_contiguous() and gate_up.shape == (tokens, 2 * inter) and gate_up.dtype == out.dtype, "silu_mul: gate_up must be [T, 2I] and out [T, I], same dtype")
    _launch("lrs_silu_mul", _dev(out, "out"), _dev(gate_up, "gate_up"), dtype_code(out.dtype), tokens, inter, 1 if interleaved else 0, _stream())


def add_into(residual: torch.Tensor, y: torch.Tensor) -> None:
    """residual (float32) += y, same shape, both contiguous."""
    _need(residual.dtype == torch.float32 and residual.shape == y.shape and residual.is_contiguous() and y.is_contiguous(), "add_into: float32 residual and y of one contiguous shape needed")
    _launch("lrs_add_into", _dev(residual, "residual"), _dev(y, "y"), dtype_code(y.dtype), residual.numel(), _stream())


@functools.lru_cache(maxsize=4096)
def gemm_lines_width(m: int, n: int, k: int) -> int:
    """The tile width (256, 192 or 128 weight rows) the many-rows kernel with slices of whole lines would take
    for out [m, n] = x [m, k] w[n, k]^T, or 0 if that kernel does not take the product."""
    return int(library().lrs_gemm_lines_width(m, n, k))


@functools.lru_cache(maxsize=4096)
def gemm_lines_splits(m: int, n: int, k: int) -> int:
    """Into how many parts the many-rows kernel with slices of whole lines divides K for a product with too few
    tiles of 256 x 128 to go round the compute units (1: the tiles as they are), or 0 if it does not take the
    product that way."""
    return int(library().lrs_gemm_lines_splits(m, n, k))


@functools.lru_cache(maxsize=4096)
def gemm_split_pays(m: int, n: int, k: int) -> bool:
    """Whether a bfloat16 product of more than 128 rows is faster by this package's many-rows kernel with K divided
    between workgroups than by the vendor library (a rule from measurements, see `lrs_gemm_lines_split_pays`)."""
    return bool(library().lrs_gemm_lines_split_pays(m, n, k))


def few_rows_capacity() -> int:
    """Most rows the few-rows product kernel takes at all (callers use it up to KernelChoice.few_rows_max)."""
    return library().lrs_gemm_skinny_capacity()


def gemm_mid_shape(n: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> tuple[int, int]:
    """(waves a workgroup, K splits) the kernel for 17..128 rows takes for a weight matrix [n, k]."""
    waves, splits = c_int(0), c_int(0)
    _check(library().lrs_gemm_mid_shape(n, k, choice.word, ctypes.addressof(waves), ctypes.addressof(splits)))
    return waves.value, splits.value


def gemm_mid_deal(m: int, n: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> tuple[int, int, int, int]:
    """(waves a workgroup, K splits, workgroups along n, how many of them have 16 rows more than 16 * waves) for a
    product of m rows (17..128) with a weight matrix [n, k]."""
    waves, splits, groups, extras = c_int(0), c_int(0), c_int(0), c_int(0)
    _check(library().lrs_gemm_mid_deal(m, n, k, choice.word, ctypes.addressof(waves), ctypes.addressof(splits), ctypes.addressof(groups),
                                       ctypes.addressof(extras)))
    return waves.value, splits.value, groups.value, extras.value


# Rows up to which callers that may use the vendor library take this package's kernel for 17..128 rows instead.
# Measured on MI355X in whole decode steps (Qwen3-8B shape): 4-6 % faster than the library's products at
# batches of 24..64; at 128 rows a layer's four products take 141 us against 169 us (and a separate gated
# activation), only the LM head is slower (320 against 279 us).
MID_ROWS_PREFERRED = 128


def gemm_mid_takes(dtype: torch.dtype, m: int, n: int, k: int, most: int = 128, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether a product of m rows (at most `most`) can go to the kernel for 17..128 rows (weights streamed
    once, activations shared through LDS), which also writes the gated activation itself."""
    return dtype == torch.bfloat16 and 16 < m <= min(most, 128) and k % 256 == 0 and n % 16 == 0 and choice.mid


def norm_begin_parts(n: int) -> int:
    """Partial sums of squares per row that gemm_mid_add_norm_begin() leaves for a norm over n columns."""
    return library().lrs_norm_begin_parts(n)


def gemm_mid_add_norm_begin(residual: torch.Tensor, a: torch.Tensor, w: torch.Tensor, norm_weight: torch.Tensor,
                            next_x: torch.Tensor, next_sumsq: torch.Tensor, choice: KernelChoice = DEFAULT_CHOICE,
                            workspace: torch.Tensor | None = None) -> None:
    """residual (float32 [M, N]) += a @ w.T for 17..128 bf16 rows, and the first half of the RMSNorm that follows:
    next_x [M, N] = bf16(residual * norm_weight), next_sumsq [norm_begin_parts(N), M] = partial sums of residual^2.
    gemm_mid_scaled() (or scale_rows()) finishes the norm."""
    m, k = a.shape
    n = w.shape[0]
    _need(gemm_mid_takes(w.dtype, m, n, k, 128, choice) and a.dtype == torch.bfloat16, "gemm_mid_add_norm_begin: takes bf16 products of 17..128 rows, K % 256 == 0, N % 16 == 0")
    _need(w.dim() == 2 and w.is_contiguous() and w.shape[1] == k, f"gemm_mid_add_norm_begin: weight must be contiguous [N, {k}]")
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and residual.shape == (m, n), f"gemm_mid_add_norm_begin: residual must be contiguous float32 [{m}, {n}]")
    _need(next_x.dtype == torch.bfloat16 and next_x.is_contiguous() and next_x.shape == (m, n), f"gemm_mid_add_norm_begin: next_x must be contiguous bf16 [{m}, {n}]")
    _need(next_sumsq.dtype == torch.float32 and next_sumsq.is_contiguous() and next_sumsq.shape == (norm_begin_parts(n), m),
          f"gemm_mid_add_norm_begin: next_sumsq must be contiguous float32 [{norm_begin_parts(n)}, {m}]")
    _need(norm_weight.is_contiguous() and norm_weight.numel() == n, f"gemm_mid_add_norm_begin: norm weight must hold {n} values")
    _launch("lrs_gemm_mid_add_norm_begin", _dev(residual, "residual"), _dev(a, "a"), _dev(w, "w"), _dev(norm_weight, "norm_weight"),
                                                 dtype_code(norm_weight.dtype), _dev(next_x, "next_x"), _dev(next_sumsq, "next_sumsq"),
                                                 m, n, k, _rows(a, "a"), choice.word, *_workspace(workspace, "gemm_mid_add_norm_begin"), _stream())


def gemm_mid_scaled(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, sumsq: torch.Tensor, eps: float, swiglu: bool = False,
                    choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """out = (the RMSNorm that `a` and `sumsq` stand for) @ w.T for 17..128 rows: a = bf16(h * norm weight) [M, K],
    sumsq [parts, M] partial sums of h^2; row r of the product is multiplied by rsqrt(sum_p sumsq[p, r] / K + eps).
    swiglu as in gemm()."""
    m, k = a.shape
    n = w.shape[0]
    _need(gemm_mid_takes(w.dtype, m, n, k, 128, choice) and a.dtype == torch.bfloat16, "gemm_mid_scaled: takes bf16 products of 17..128 rows, K % 256 == 0, N % 16 == 0")
    _need(w.dim() == 2 and w.is_contiguous() and w.shape[1] == k, f"gemm_mid_scaled: weight must be contiguous [N, {k}]")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm_mid_scaled: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    _need(out.dtype in (torch.bfloat16, torch.float32) and not (swiglu and out.dtype != torch.bfloat16), "gemm_mid_scaled: output must be bf16, or float32 without swiglu")
    _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous() and eps > 0, f"gemm_mid_scaled: sumsq must be float32 [parts, {m}] and eps positive")
    mode = OUT_STORE if out.dtype == torch.bfloat16 else OUT_STORE_F32
    _launch("lrs_gemm_mid_scaled", _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), m, n, k, _rows(a, "a"), _rows(out, "out"),
                                         int(swiglu), _dev(sumsq, "sumsq"), sumsq.shape[0], eps, choice.word,
                                         *_workspace(workspace, "gemm_mid_scaled"), _stream())


def _int_vector(t: torch.Tensor, name: str, at_least: int) -> int:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= at_least, f"{name} must be contiguous int32 with at least {at_least} elements")
    return _dev(t, name)


def advance_decode(token_ids: torch.Tensor, positions: torch.Tensor, token_request: torch.Tensor, seq_lens: torch.Tensor,
                   chosen: torch.Tensor, real_rows: torch.Tensor, draws: torch.Tensor | None = None) -> None:
    """A decode step's metadata moved on to the next step, on the device: the first real_rows[0] rows
    take the tokens in `chosen`, move one position on, lengthen their requests by one and (with
    `draws`, the counters of seeded sampling) count one more draw."""
    rows = token_ids.numel()
    _launch("lrs_advance_decode", _int_vector(token_ids, "token_ids", rows), _int_vector(positions, "positions", rows),
                                        _int_vector(token_request, "token_request", rows), _int_vector(seq_lens, "seq_lens", 1),
                                        _int_vector(chosen, "chosen", rows), None if draws is None else _int_vector(draws, "draws", rows),
                                        _int_vector(real_rows, "real_rows", 1), rows, _stream())


def advance_slots(slots: torch.Tensor, positions: torch.Tensor, token_request: torch.Tensor, block_table: torch.Tensor,
                  page_size: int, real_rows: torch.Tensor) -> None:
    """The cache slots of the (already advanced) positions of the first real_rows[0] rows, from the block table."""
    rows = slots.numel()
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "advance_slots: block_table must be int32 [R, blocks]")
    _launch("lrs_advance_slots", _int_vector(slots, "slots", rows), _int_vector(positions, "positions", rows),
                                       _int_vector(token_request, "token_request", rows), _dev(block_table, "block_table"),
                                       block_table.stride(0), page_size, _int_vector(real_rows, "real_rows", 1), rows, _stream())


def step_prepare_summary_size() -> int:
    return library().lrs_step_prepare_summary_size()


def step_prepare(meta, offsets, entries: int, packed, tokens_at: int, wants_at: int, pad_to: int, trash_slot: int, tables,
                 groups: int, max_blocks: int, page_size: int, query_group: int, summary) -> None:
    """Fill a step's metadata in the staging buffer `meta` (a numpy int32 view of pinned memory) on the host: see
    csrc/prepare.hip.  `packed` (numpy int32) holds, `entries` values each, the entries' state slots, context lengths,
    token counts and numbers of wanted places, then from `tokens_at` all tokens and from `wants_at` all wanted places;
    `offsets` (numpy int64) where each array lies in `meta`; `tables` a ctypes array of the host block tables' addresses;
    `summary` (numpy int32) takes T, R, logit rows, query groups, largest group, longest portion, longest context and
    the single rows at the step's head."""
    base = packed.ctypes.data
    code = library().lrs_step_prepare(meta.ctypes.data, offsets.ctypes.data, entries, base, base + 4 * entries, base + 8 * entries,
                                      base + 4 * tokens_at, base + 12 * entries, base + 4 * wants_at, pad_to, trash_slot, groups,
                                      ctypes.cast(tables, c_void_p), max_blocks, page_size, query_group, summary.ctypes.data)
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())


def fill_i32(dst: torch.Tensor, value: int) -> None:
    _need(dst.dtype == torch.int32 and dst.is_contiguous(), "fill_i32: int32 contiguous tensor needed")
    _launch("lrs_fill_i32", _dev(dst, "dst"), value, dst.numel(), _stream())


def scatter_i32(dst: torch.Tensor, pairs: torch.Tensor, count: int, first: int = 0) -> None:
    """dst.view(-1)[offset_i] = value_i for the `count` (offset, value) pairs that lie in `pairs` (int32, on the device)
    from element `first` on.  The caller has checked that every offset lies inside dst."""
    _need(dst.dtype == torch.int32 and dst.is_contiguous() and pairs.dtype == torch.int32 and pairs.is_contiguous()
          and first >= 0 and first % 2 == 0 and 0 < 2 * count <= pairs.numel() - first,
          "scatter_i32: int32 contiguous tensors and 2 * count values in pairs from an even element on needed")
    _launch("lrs_scatter_i32", _dev(dst, "dst"), _dev(pairs, "pairs") + 4 * first, count, _stream())


def gather_rows(out: torch.Tensor, x: torch.Tensor, rows: torch.Tensor) -> None:
    n_rows, hidden = out.shape
    _need(out.is_contiguous() and x.is_contiguous() and x.shape[1] == hidden, "gather_rows: shapes disagree")
    _need(rows.dtype == torch.int32 and rows.numel() >= n_rows, "gather_rows: rows must be int32")
    _launch("lrs_gather_rows", _dev(out, "out", torch.float32), _dev(x, "x", torch.float32), _dev(rows, "rows"), n_rows, hidden, _stream())


# ------------------------------------------------------------------- gemm
def gemm_fuses_norm(dtype: torch.dtype, m: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm() can take the float32 residual stream and normalise it on the way in."""
    return dtype == torch.bfloat16 and m <= choice.few_rows_max and k % 8 == 0


def gemm_norm_fusion_pays(n: int) -> bool:
    """Every workgroup of the fused kernel normalises the whole input again, so the fusion costs
    more than the norm kernel it saves once the weight matrix has many rows (measured on MI355X:
    even at 6144 rows it only breaks even)."""
    return n <= 4096


def gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None, accumulate: bool = False,
         swiglu: bool = False, norm_weight: torch.Tensor | None = None, eps: float = 0.0, rows: torch.Tensor | None = None,
         count: int | None = None, choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """out = a @ w.T (+ bias).  `accumulate` adds into a float32 `out` instead of storing.

    workspace: the caller's own device memory (gemm_workspace_bytes()) for the sums of K splits, which some shapes
    leave for a second kernel; without it the process-wide one is used, which is safe on one stream only.

    norm_weight: `a` is the float32 residual stream [*, K]; the product is taken of its RMSNorm
    (weight norm_weight, eps), of the `count` rows listed in `rows` if given, else of its first rows.
    swiglu: `w` holds gate and up rows interleaved in groups of 8; out [M, N/2] = silu(gate) * up.
    """
    n, k = w.shape
    lda, ldc = _rows(a, "a"), _rows(out, "out")
    _need(w.dim() == 2 and w.is_contiguous() and a.shape[1] == k, f"gemm: weight must be contiguous [N, {a.shape[1]}], got {tuple(w.shape)}")
    normed = norm_weight is not None
    if normed:
        m = count if rows is not None else out.shape[0]
        _need(a.dtype == torch.float32 and gemm_fuses_norm(w.dtype, m, k, choice), f"gemm: the fused norm input needs a float32 input, bf16 weights and at most {choice.few_rows_max} rows")
        _need(norm_weight.numel() == k and norm_weight.is_contiguous() and eps > 0, "gemm: norm weight must hold K values and eps be positive")
        if rows is None:
            _need(a.shape[0] >= m, "gemm: input has fewer rows than the output")
        else:
            _need(rows.dtype == torch.int32 and rows.numel() >= m and rows.is_contiguous(), "gemm: rows must be int32")
    else:
        m = a.shape[0]
        _need(rows is None, "gemm: a row gather needs the fused norm input")
        _need(a.dtype == w.dtype, f"gemm: a is {a.dtype} but w is {w.dtype}")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
        mode = OUT_ADD_F32
    elif out.dtype == w.dtype:
        mode = OUT_STORE
    else:
        _need(out.dtype == torch.float32, "gemm: output must be of the weight dtype or float32")
        mode = OUT_STORE_F32
    if bias is not None:
        _need(bias.numel() == n and bias.dtype == w.dtype and bias.is_contiguous(), "gemm: bias must hold N values of the weight dtype")
    if swiglu:
        _need(w.dtype == torch.bfloat16 and n % 16 == 0 and k % 8 == 0 and bias is None and mode == OUT_STORE, "gemm: swiglu needs bf16, N % 16 == 0, K % 8 == 0, no bias, a stored output")
    _launch("lrs_gemm", _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), None if bias is None else _dev(bias, "bias"),
                              dtype_code(w.dtype), m, n, k, lda, ldc, None if rows is None else _dev(rows, "rows"),
                              None if not normed else _dev(norm_weight, "norm_weight"), dtype_code(norm_weight.dtype) if normed else 0,
                              eps, 1 if swiglu else 0, choice.word, *_workspace(workspace, "gemm"), _stream())


def gemm_lines_add_rmsnorm(residual: torch.Tensor, a: torch.Tensor, w: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                           normed: torch.Tensor, workspace: torch.Tensor | None = None) -> None:
    """residual (float32 [M, N]) += a @ w.T for more than 128 bf16 rows of a shape that gemm_lines_splits() takes, and
    normed [M, N] = RMSNorm(residual) with `norm_weight` and `eps`: the product with its K divided between workgroups,
    and one kernel that adds up their sums, adds them to the residual stream and normalises the rows."""
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape == (n, k) and w.is_contiguous() and m > 128
          and gemm_lines_splits(m, n, k) >= 1, "gemm_lines_add_rmsnorm: takes bf16 products of more than 128 rows that gemm_lines_splits() takes")
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and residual.shape == (m, n), f"gemm_lines_add_rmsnorm: residual must be contiguous float32 [{m}, {n}]")
    _need(normed.is_contiguous() and normed.shape == (m, n), f"gemm_lines_add_rmsnorm: normed must be contiguous [{m}, {n}]")
    _need(norm_weight.is_contiguous() and norm_weight.numel() == n and eps > 0 and n % 4 == 0 and n <= 8192,
          f"gemm_lines_add_rmsnorm: the norm weight must hold {n} values, eps be positive and N a multiple of 4 up to 8192")
    _launch("lrs_gemm_lines_add_rmsnorm", _dev(residual, "residual"), _dev(a, "a"), _dev(w, "w"), m, n, k, _rows(a, "a"),
            _dev(norm_weight, "norm_weight"), dtype_code(norm_weight.dtype), eps, _dev(normed, "normed"), dtype_code(normed.dtype),
            *_workspace(workspace, "gemm_lines_add_rmsnorm"), _stream())


def library_gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor) -> None:
    """out [M, N] = a [M, K] @ w[N, K].T by the vendor's matrix library (bfloat16 inputs, float32 sums; out bfloat16
    or float32): for products of more rows than this package's own kernels are made for."""
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == k and w.is_contiguous(),
          f"library_gemm: a and w must be bfloat16, w contiguous [N, {k}]")
    _need(out.shape == (m, n) and out.dtype in (torch.bfloat16, torch.float32), f"library_gemm: out must be bfloat16 or float32 [{m}, {n}]")
    _launch("lrs_library_gemm", _dev(out, "out"), 1 if out.dtype == torch.float32 else 0, _dev(a, "a"), _dev(w, "w"), m, n, k,
                                      _rows(a, "a"), _rows(out, "out"), _stream())


NORM_CHAIN_MAX_ROWS = 16


def gemm_chains_norm(dtype: torch.dtype, m: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm_norm_chain() takes a product of m rows over k with weights of `dtype`."""
    return dtype == torch.bfloat16 and m <= min(NORM_CHAIN_MAX_ROWS, choice.few_rows_max) and k % 8 == 0


def norm_chain_parts(n: int) -> int:
    """Partial sums of squares per row that a product of n output columns leaves for the next norm."""
    return library().lrs_gemm_norm_chain_parts(n)


def gemm_norm_chain(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
                    accumulate: bool = False, swiglu: bool = False,
                    in_sumsq: torch.Tensor | None = None, in_eps: float = 0.0,
                    next_x: torch.Tensor | None = None, next_sumsq: torch.Tensor | None = None,
                    next_weight: torch.Tensor | None = None, choice: KernelChoice = DEFAULT_CHOICE) -> None:
    """out = a @ w.T (+ bias) for at most 16 bf16 rows, with an RMSNorm taken apart around it.

    in_sumsq [parts, M] float32: `a` holds bf16(h * norm weight); row r of the product is multiplied
    by rsqrt(sum_p in_sumsq[p, r] / K + in_eps), which completes the norm.
    next_x [M, N] bf16, next_sumsq [norm_chain_parts(N), M] float32, next_weight [N] (needs
    `accumulate`): besides adding into `out`, write bf16(out_new * next_weight) and the partial sums
    of out_new^2, the input of the next product called with in_sumsq."""
    n, k = w.shape
    m = a.shape[0]
    lda, ldc = _rows(a, "a"), _rows(out, "out")
    _need(w.dim() == 2 and w.is_contiguous() and a.shape[1] == k, f"gemm_norm_chain: weight must be contiguous [N, {a.shape[1]}], got {tuple(w.shape)}")
    _need(a.dtype == torch.bfloat16 and gemm_chains_norm(w.dtype, m, k, choice), "gemm_norm_chain: needs bf16 input and weights, at most 16 rows, K % 8 == 0")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm_norm_chain: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm_norm_chain: accumulation needs a float32 output")
        mode = OUT_ADD_F32
    elif out.dtype == w.dtype:
        mode = OUT_STORE
    else:
        _need(out.dtype == torch.float32, "gemm_norm_chain: output must be bf16 or float32")
        mode = OUT_STORE_F32
    if bias is not None:
        _need(bias.numel() == n and bias.dtype == w.dtype and bias.is_contiguous(), "gemm_norm_chain: bias must hold N values of the weight dtype")
    if swiglu:
        _need(n % 16 == 0 and bias is None and mode == OUT_STORE, "gemm_norm_chain: swiglu needs N % 16 == 0, no bias, a stored output")
    parts = 0
    if in_sumsq is not None:
        _need(in_sumsq.dtype == torch.float32 and in_sumsq.dim() == 2 and in_sumsq.shape[1] == m and in_sumsq.is_contiguous() and in_eps > 0,
              f"gemm_norm_chain: in_sumsq must be contiguous float32 [parts, {m}] and in_eps positive")
        parts = in_sumsq.shape[0]
    if next_x is not None:
        _need(accumulate and not swiglu, "gemm_norm_chain: only a product that adds into the residual stream can feed the next norm")
        _need(next_x.dtype == torch.bfloat16 and next_x.shape == (m, n) and next_x.is_contiguous(), f"gemm_norm_chain: next_x must be contiguous bf16 [{m}, {n}]")
        _need(next_sumsq is not None and next_sumsq.dtype == torch.float32 and next_sumsq.shape == (norm_chain_parts(n), m) and next_sumsq.is_contiguous(),
              f"gemm_norm_chain: next_sumsq must be contiguous float32 [{norm_chain_parts(n)}, {m}]")
        _need(next_weight is not None and next_weight.numel() == n and next_weight.is_contiguous(), "gemm_norm_chain: next_weight must hold N values")
    _launch("lrs_gemm_norm_chain", 
        _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), None if bias is None else _dev(bias, "bias"), m, n, k, lda, ldc,
        1 if swiglu else 0, None if in_sumsq is None else _dev(in_sumsq, "in_sumsq"), parts, in_eps,
        None if next_x is None else _dev(next_x, "next_x"), None if next_x is None else _dev(next_sumsq, "next_sumsq"),
        None if next_x is None else _dev(next_weight, "next_weight"), dtype_code(next_weight.dtype) if next_x is not None else 0,
        choice.word, _stream())


def scale_rows(out: torch.Tensor, x: torch.Tensor, sumsq: torch.Tensor, eps: float) -> None:
    """out[r] = x[r] * rsqrt(sum_p sumsq[p, r] / hidden + eps): completes a norm that gemm_norm_chain() began."""
    m, hidden = x.shape
    _need(x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.shape == x.shape and x.is_contiguous() and out.is_contiguous(),
          "scale_rows: x and out must be contiguous bf16 of one shape")
    _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous(), f"scale_rows: sumsq must be float32 [parts, {m}]")
    _launch("lrs_scale_rows", _dev(out, "out"), _dev(x, "x"), _dev(sumsq, "sumsq"), sumsq.shape[0], m, hidden, eps, _stream())


# -------------------------------------------------------------- attention
def attention(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
              token_request: torch.Tensor, positions: torch.Tensor, nq: int, scale: float, window: int = 0) -> None:
    """out [T, nq*d]; q [T, >= nq*d] (leading nq*d columns of each row); key pages [P, nkv, page, d],
    value pages [P, nkv, d, page]."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    _need(v_pages.shape == (k_pages.shape[0], nkv, d, page_size), "attention: key pages must be [P, nkv, page, d] and value pages [P, nkv, d, page]")
    _need(out.shape[1] == nq * d and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention: q/out widths do not match nq*d")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention: {name} must be int32 [T]")
    _launch("lrs_attention", 
        _dev(out, "out"), _rows(out, "out"), _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
        _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"), _dev(positions, "positions"),
        dtype_code(q.dtype), tokens, nq, nkv, d, page_size, scale, window, _stream())


DECODE_HEAD_DIMS = (32, 64, 96, 128, 192)


def attention_decode_supported(dtype: torch.dtype, nq: int, nkv: int, d: int, page_size: int) -> bool:
    """Whether the matrix-core decode kernel takes this shape (else use attention())."""
    return dtype == torch.bfloat16 and d in DECODE_HEAD_DIMS and page_size % 16 == 0 and nq // nkv <= 16


@dataclass
class DecodePrepare:
    """What attention_decode() does to the raw q/k/v rows when it stands in for qk_prep(): per-head
    RMSNorm of q and k (weights None: none), rotation of the whole head by cos/sin [T, d/2] (None:
    none), and the write of the new key and value into the pages (kv_heads = the number of kv heads
    held in the rows; 0 for a layer that reads another layer's pages)."""
    q_weight: torch.Tensor | None
    k_weight: torch.Tensor | None
    eps: float
    cos: torch.Tensor | None
    sin: torch.Tensor | None
    kv_heads: int


def decode_prepare_supported(d: int, rotates: bool) -> bool:
    """Whether attention_decode() can do qk_prep()'s work for heads of d dims (it rotates pairs that
    lie 32-dim chunks apart: d a multiple of 64)."""
    return not rotates or d % 64 == 0


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                     token_request: torch.Tensor, positions: torch.Tensor, nq: int, scale: float, window: int = 0, splits: int = 1,
                     part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None, max_context: int | None = None,
                     prepare: "DecodePrepare | None" = None, form: int = 0) -> None:
    """attention() for a step with one query token per request, bfloat16 only; the keys of a token
    are divided between `splits` workgroups whose partial results meet in part_o / part_ml.

    prepare: `q` holds the raw rows of the q/k/v product and the kernel also does what qk_prep()
    does (see DecodePrepare); without it q, and the pages, must have been through qk_prep()."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention_decode: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    _need(v_pages.shape == (k_pages.shape[0], nkv, d, page_size), "attention_decode: key pages must be [P, nkv, page, d] and value pages [P, nkv, d, page]")
    _need(attention_decode_supported(q.dtype, nq, nkv, d, page_size), f"attention_decode: unsupported shape nq={nq} nkv={nkv} d={d} page={page_size} {q.dtype}")
    _need(out.shape[1] == nq * d and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention_decode: q/out widths do not match nq*d")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention_decode: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention_decode: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention_decode: {name} must be int32 [T]")
    if splits > 1:
        _need(part_o is not None and part_o.dtype == torch.float32 and part_o.is_contiguous() and part_o.numel() >= tokens * nq * splits * d, "attention_decode: part_o too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous() and part_ml.numel() >= tokens * nq * splits * 2, "attention_decode: part_ml too small")
    fused = [0, None, None, 0, 0.0, None, None, 0]
    if prepare is not None:
        _need(decode_prepare_supported(d, prepare.cos is not None), f"attention_decode: cannot rotate heads of {d} dims itself")
        _need((prepare.q_weight is None) == (prepare.k_weight is None), "attention_decode: q and k norm weights must come together")
        _need(prepare.kv_heads in (0, nkv) and q.shape[1] >= (nq + 2 * prepare.kv_heads) * d, "attention_decode: q rows must hold the q heads and kv_heads (0 or all) k and v heads")
        for name, w in (("q_weight", prepare.q_weight), ("k_weight", prepare.k_weight)):
            _need(w is None or (w.numel() == d and w.is_contiguous() and w.dtype == prepare.q_weight.dtype), f"attention_decode: {name} must hold head_dim values")
        for name, t in (("cos", prepare.cos), ("sin", prepare.sin)):
            _need((t is None) == (prepare.cos is None) and (t is None or (t.dtype == torch.float32 and t.shape == (tokens, d // 2) and t.is_contiguous())),
                  f"attention_decode: {name} must be float32 [{tokens}, {d // 2}]")
        normed = prepare.q_weight is not None
        _need(not normed or prepare.eps > 0, "attention_decode: eps must be positive")
        fused = [1, _dev(prepare.q_weight, "q_weight") if normed else None, _dev(prepare.k_weight, "k_weight") if normed else None,
                 dtype_code(prepare.q_weight.dtype) if normed else 0, prepare.eps,
                 None if prepare.cos is None else _dev(prepare.cos, "cos"), None if prepare.sin is None else _dev(prepare.sin, "sin"), prepare.kv_heads]
    _launch("lrs_attention_decode", 
        _dev(out, "out"), _rows(out, "out"), None if splits == 1 else _dev(part_o, "part_o"), None if splits == 1 else _dev(part_ml, "part_ml"),
        _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table"), block_table.stride(0),
        _dev(token_request, "token_request"), _dev(positions, "positions"), tokens,
        block_table.shape[1] * page_size if max_context is None else max_context, nq, nkv, d, page_size, scale, window, splits,
        form, *fused, _stream())


def attention_prefill(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                      token_request: torch.Tensor, positions: torch.Tensor, qblock_token0: torch.Tensor, qblock_count: torch.Tensor,
                      nq: int, scale: float, window: int = 0, max_count: int | None = None, max_context: int | None = None,
                      splits: int = 1, part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None,
                      prepare: "DecodePrepare | None" = None) -> None:
    """attention() on matrix cores for any bfloat16 step.  qblock_token0 / qblock_count list groups of at
    most attention_prefill_group() consecutive tokens of one request that together cover every token of
    the step once; `max_count` is the largest count among them (the group limit if not given) and
    `max_context` the longest context (position + 1) of any token (what the block table can hold if not given).
    splits > 1 divides every group's keys between that many workgroups (few queries over long contexts);
    their partial results meet in part_o [T, nq * splits * d] and part_ml [T, nq * splits * 2] float32.
    prepare (where attention_prefill_prepares(d)): `q` holds the raw q heads of the q/k/v product, and the kernel gives
    them their norm and rotation itself (q_weight, eps, cos, sin of DecodePrepare; kv_heads 0: the keys and values are in
    the pages already, from qk_prep(skip_q=True))."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention_prefill: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    _need(v_pages.shape == (k_pages.shape[0], nkv, d, page_size), "attention_prefill: key pages must be [P, nkv, page, d] and value pages [P, nkv, d, page]")
    _need(attention_decode_supported(q.dtype, nq, nkv, d, page_size), f"attention_prefill: unsupported shape nq={nq} nkv={nkv} d={d} page={page_size} {q.dtype}")
    _need(out.shape[1] == nq * d and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention_prefill: q/out widths do not match nq*d")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention_prefill: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention_prefill: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention_prefill: {name} must be int32 [T]")
    n_blocks = qblock_token0.numel()
    _need(n_blocks > 0 and qblock_count.numel() == n_blocks and qblock_token0.dtype == qblock_count.dtype == torch.int32
          and qblock_token0.is_contiguous() and qblock_count.is_contiguous(), "attention_prefill: query blocks must be two int32 vectors of one length")
    _need(1 <= splits <= 64, f"attention_prefill: splits must be 1..64, got {splits}")
    if splits > 1:
        _need(part_o is not None and part_o.dtype == torch.float32 and part_o.is_contiguous() and part_o.numel() >= tokens * nq * splits * d, "attention_prefill: part_o too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous() and part_ml.numel() >= tokens * nq * splits * 2, "attention_prefill: part_ml too small")
    fused = [0, None, 0, 0.0, None, None]
    if prepare is not None:
        _need(attention_prefill_prepares(d), f"attention_prefill: heads of {d} dims must come prepared")
        _need(prepare.kv_heads == 0, "attention_prefill: prepares the queries only (kv_heads must be 0)")
        w = prepare.q_weight
        _need(w is None or (w.numel() == d and w.is_contiguous() and prepare.eps > 0), "attention_prefill: q_weight must hold head_dim values, eps be positive")
        for name, t in (("cos", prepare.cos), ("sin", prepare.sin)):
            _need((t is None) == (prepare.cos is None) and (t is None or (t.dtype == torch.float32 and t.dim() == 2 and t.shape[0] >= tokens
                                                                       and t.shape[1] == d // 2 and t.is_contiguous())),
                  f"attention_prefill: {name} must be float32 [{tokens}, {d // 2}]")
        fused = [1, None if w is None else _dev(w, "q_weight"), 0 if w is None else dtype_code(w.dtype), prepare.eps,
                 None if prepare.cos is None else _dev(prepare.cos, "cos"), None if prepare.sin is None else _dev(prepare.sin, "sin")]
    _launch("lrs_attention_prefill", 
        _dev(out, "out"), _rows(out, "out"), _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
        _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"), _dev(positions, "positions"),
        _dev(qblock_token0, "qblock_token0"), _dev(qblock_count, "qblock_count"), n_blocks,
        attention_prefill_group() if max_count is None else max_count,
        block_table.shape[1] * page_size if max_context is None else max_context, nq, nkv, d, page_size, scale, window,
        tokens, splits, None if splits == 1 else _dev(part_o, "part_o"), None if splits == 1 else _dev(part_ml, "part_ml"), *fused, _stream())


def attention_prefill_prepares(d: int) -> bool:
    """Whether attention_prefill() can take raw q heads of d dims and prepare them itself."""
    return bool(library().lrs_attention_prefill_prepares(d))


def compute_units() -> int:
    """Compute units of the device (workgroups of one kernel that can start at the same time, per occupancy)."""
    return library().lrs_compute_units()


def attention_prefill_group(tokens: int | None = None, longest: int = 0) -> int:
    """Most tokens in one query group of attention_prefill(); with `tokens`, the group size that
    serves a step of that many tokens best (smaller groups fill the chip when there are few), given the
    longest context (position + 1) among them, if known (larger groups pay earlier behind a long context)."""
    if tokens is None:
        return library().lrs_attention_prefill_group()
    return library().lrs_attention_prefill_group_for(tokens, longest)


# --------------------------------------------------------------- sampling
_choose_scratch: dict = {}


def choose_tokens(out: torch.Tensor, logits: torch.Tensor, temperature=None, seeds=None, counters=None,
                  out_address: int | None = None, filtered: bool = False) -> None:
    """One token per row of logits into `out`, int32 [R] on the device; or, with `out_address` (from
    pinned_device_address(out)), into pinned host memory that the kernel writes directly and the
    host reads after synchronising the stream.  A row that holds a value that is not finite gets -1
    (the reference refuses such logits, mini_llm/sampling.py:104-113); `filtered`: filter_logits() has
    been over the rows, so those of positive temperature may hold -inf."""
    rows, vocab = logits.shape
    _need(out.dtype == torch.int32 and out.numel() >= rows and out.is_contiguous(), "choose_tokens: out must be int32 [R]")
    stride = _rows(logits, "logits")
    if out_address is None:
        out_pointer = _dev(out, "out")
    else:
        _need(not out.is_cuda, "choose_tokens: out_address goes with a pinned host tensor")
        out_pointer = out_address + out.storage_offset() * out.element_size()
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "choose_tokens: temperature must be float32 [R]")
        _need(seeds is not None and seeds.dtype == torch.int64 and seeds.numel() >= rows, "choose_tokens: seeds must be int64 [R]")
        _need(counters is not None and counters.dtype == torch.int32 and counters.numel() >= rows, "choose_tokens: counters must be int32 [R]")
    args = (None if temperature is None else _dev(temperature, "temperature"), None if temperature is None else _dev(seeds, "seeds"),
            None if temperature is None else _dev(counters, "counters"))
    if vocab >= 16384:   # large vocabulary: many workgroups per row, then one to pick among their results
        parts = -(-vocab // 4096)
        key = (logits.device, rows, parts)
        scratch = _choose_scratch.get(key)
        if scratch is None:
            scratch = _choose_scratch[key] = (torch.empty(rows * parts, dtype=torch.float32, device=logits.device),
                                              torch.empty(rows * parts, dtype=torch.int32, device=logits.device))
        _launch("lrs_choose_tokens_split", out_pointer, _dev(logits, "logits", torch.float32), stride, rows, vocab, *args,
                                                 _dev(scratch[0], "part_value"), _dev(scratch[1], "part_index"), parts, int(bool(filtered)), _stream())
        return
    _launch("lrs_choose_tokens", out_pointer, _dev(logits, "logits", torch.float32), stride, rows, vocab, *args, int(bool(filtered)), _stream())


def choose_tokens_static(out: torch.Tensor, logits: torch.Tensor, parts: int, temperature=None, seeds=None, counters=None,
                         filtered: bool = False) -> None:
    """choose_tokens() in its two-pass form (`parts` slices a row) for callers that must not allocate: the
    slices' results go to a fixed array inside the library (rows * parts at most
    lrs_choose_tokens_static_max_parts()), so nothing is allocated here or there.  Calls that overlap on
    one GPU share that array and race."""
    rows, vocab = logits.shape
    _need(out.dtype == torch.int32 and out.numel() >= rows and out.is_contiguous(), "choose_tokens_static: out must be int32 [R]")
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "choose_tokens_static: temperature must be float32 [R]")
        _need(seeds is not None and seeds.dtype == torch.int64 and seeds.numel() >= rows, "choose_tokens_static: seeds must be int64 [R]")
        _need(counters is not None and counters.dtype == torch.int32 and counters.numel() >= rows, "choose_tokens_static: counters must be int32 [R]")
    _launch("lrs_choose_tokens_static", 
        _dev(out, "out"), _dev(logits, "logits", torch.float32), _rows(logits, "logits"), rows, vocab,
        None if temperature is None else _dev(temperature, "temperature"), None if temperature is None else _dev(seeds, "seeds"),
        None if temperature is None else _dev(counters, "counters"), parts, int(bool(filtered)), _stream())


def filter_logits(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor | None, top_p: torch.Tensor | None) -> None:
    rows, vocab = logits.shape
    stride = _rows(logits, "logits")
    _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "filter_logits: temperature must be float32 [R]")
    if top_k is not None:
        _need(top_k.dtype == torch.int32 and top_k.numel() >= rows, "filter_logits: top_k must be int32 [R]")
    if top_p is not None:
        _need(top_p.dtype == torch.float32 and top_p.numel() >= rows, "filter_logits: top_p must be float32 [R]")
    _launch("lrs_filter_logits", _dev(logits, "logits", torch.float32), stride, rows, vocab, _dev(temperature, "temperature"),
                                       None if top_k is None else _dev(top_k, "top_k"), None if top_p is None else _dev(top_p, "top_p"), _stream())
