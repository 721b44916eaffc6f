"""Host side of the segment-program copy kernels.

A ``SegmentProgram`` is a shard layout's whole copy compiled once into
device-resident tables (``mfsdp_segment_program_create``) and replayed with one
kernel launch per buffer.  The builders below turn the reference's shard
metadata (``ShardPlan.rank_segments``, ``ManagedParam.offset/end``) into
runs for each copy of the path:

==========================  =====================================================
builder                     reference loops it replaces
==========================  =====================================================
``pack_program``            ``_pack_full_tensor_by_rank_segments`` (runtime/flat_buffer.py:1304-1316)
                            + zero-padded staging (runtime/collectives.py:236-237)
``unpack_program``          un-pad (runtime/collectives.py:264-272)
                            + ``_unpack_rank_shards_to_full_tensor`` (runtime/flat_buffer.py:1318-1333)
``local_segments_program``  ``_copy_local_rank_segments`` (runtime/collectives.py:495-503)
``grad_fill_program``       ``fill_reduce_scatter_input`` (runtime/grad_bucket.py:71-116, 200-225)
``compact_owner_program``   ``_fill_compact_owner_reduce_scatter_input`` (runtime/flat_buffer.py:1232-1252)
==========================  =====================================================
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import numpy as np
import torch

from .. import _lib

RUN_DTYPE = np.dtype(
    [
        ("src_off", "<i8"),
        ("dst_off", "<i8"),
        ("row_len", "<i8"),
        ("rows", "<i8"),
        ("src_stride", "<i8"),
        ("dst_stride", "<i8"),
        ("src_id", "<i4"),
        ("reserved", "<i4"),
    ]
)
assert RUN_DTYPE.itemsize == ctypes.sizeof(_lib.CopyRun)

_CONVERT_CODES = {
    (torch.bfloat16, torch.float32): _lib.CONVERT_BF16_TO_F32,
    (torch.float32, torch.bfloat16): _lib.CONVERT_F32_TO_BF16,
    (torch.float16, torch.float32): _lib.CONVERT_F16_TO_F32,
    (torch.float32, torch.float16): _lib.CONVERT_F32_TO_F16,
}
CONVERTIBLE = frozenset(_CONVERT_CODES)  # (source dtype, destination dtype) pairs a program or a cast can convert


def make_runs(src_off, dst_off, row_len, src_id=0) -> np.ndarray:
    """Plain (one-row) runs from parallel arrays of element offsets."""
    src_off = np.asarray(src_off, dtype=np.int64).reshape(-1)
    runs = np.zeros(src_off.shape[0], dtype=RUN_DTYPE)
    runs["src_off"] = src_off
    runs["dst_off"] = np.asarray(dst_off, dtype=np.int64).reshape(-1)
    runs["row_len"] = np.asarray(row_len, dtype=np.int64).reshape(-1)
    runs["rows"] = 1
    runs["src_id"] = src_id
    return runs


def fill_runs_for_gaps(written: np.ndarray, dst_numel: int) -> np.ndarray:
    """Zero-fill runs for every destination element no run of ``written``
    touches (the pad tails the reference clears with ``new_zeros`` /
    ``packed.zero_()``)."""
    starts = written["dst_off"].astype(np.int64)
    ends = starts + written["row_len"].astype(np.int64)
    if np.any(written["rows"] != 1):
        raise ValueError("fill_runs_for_gaps expects one-row runs.")
    order = np.argsort(starts, kind="stable")
    starts, ends = starts[order], ends[order]
    if starts.size and np.any(starts[1:] < ends[:-1]):
        raise ValueError("destination ranges of a segment program overlap.")
    gap_starts = np.concatenate(([0], ends)) if starts.size else np.array([0], dtype=np.int64)
    gap_ends = np.concatenate((starts, [dst_numel])) if starts.size else np.array([dst_numel], dtype=np.int64)
    keep = gap_ends > gap_starts
    return make_runs(np.zeros(int(keep.sum()), dtype=np.int64), gap_starts[keep], (gap_ends - gap_starts)[keep], src_id=-1)


def merge_runs(runs: np.ndarray) -> np.ndarray:
    """``mfsdp_merge_segment_runs``: consecutive equal-length segments at a
    constant pitch collapse into 2-D strided runs."""
    runs = np.ascontiguousarray(runs, dtype=RUN_DTYPE)
    if runs.shape[0] == 0:
        return runs
    out = np.zeros_like(runs)
    n = _lib.lib().mfsdp_merge_segment_runs(
        runs.ctypes.data_as(ctypes.POINTER(_lib.CopyRun)), runs.shape[0], out.ctypes.data_as(ctypes.POINTER(_lib.CopyRun))
    )
    return out[:n].copy()


class SegmentProgram:
    """Owns one ``mfsdp_segment_program``.  ``run`` is one kernel launch on
    the current HIP stream (one per block of 128 sources and per vector width
    in use); it neither allocates nor synchronises."""

    def __init__(
        self,
        runs: np.ndarray,
        src_numels: Sequence[int],
        dst_numel: int,
        *,
        src_dtype: torch.dtype,
        dst_dtype: torch.dtype | None = None,
        device: torch.device | str | int = "cuda",
        merge: bool = True,
    ) -> None:
        dst_dtype = dst_dtype or src_dtype
        if src_dtype == dst_dtype:
            convert, elem_bytes = _lib.CONVERT_NONE, torch.empty((), dtype=src_dtype).element_size()
        elif (src_dtype, dst_dtype) in _CONVERT_CODES:
            convert, elem_bytes = _CONVERT_CODES[(src_dtype, dst_dtype)], 0
        else:
            raise RuntimeError(f"segment programs convert bfloat16 / float16 <-> float32 only, got {src_dtype} -> {dst_dtype}.")
        self.src_dtype, self.dst_dtype = src_dtype, dst_dtype
        self.src_numels = tuple(int(n) for n in src_numels)
        self.dst_numel = int(dst_numel)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("segment programs run on a HIP device.")
        runs = merge_runs(runs) if merge else np.ascontiguousarray(runs, dtype=RUN_DTYPE)
        self.num_runs = int(runs.shape[0])
        numels = (ctypes.c_int64 * max(1, len(self.src_numels)))(*self.src_numels)
        handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            _lib.check(
                _lib.lib().mfsdp_segment_program_create(
                    runs.ctypes.data_as(ctypes.POINTER(_lib.CopyRun)),
                    runs.shape[0],
                    numels,
                    len(self.src_numels),
                    self.dst_numel,
                    convert,
                    elem_bytes,
                    ctypes.byref(handle),
                )
            )
        self._handle = handle
        self.bytes_moved = int(_lib.lib().mfsdp_segment_program_bytes(handle))
        self._src_array = (ctypes.c_void_p * max(1, len(self.src_numels)))()

    def run(self, srcs: Sequence[torch.Tensor], dst: torch.Tensor) -> torch.Tensor:
        if self._handle is None:
            raise RuntimeError("segment program was destroyed.")
        if len(srcs) != len(self.src_numels):
            raise RuntimeError(f"segment program expects {len(self.src_numels)} sources, got {len(srcs)}.")
        _check_tensor(dst, self.dst_dtype, self.dst_numel, "destination")
        for i, (t, n) in enumerate(zip(srcs, self.src_numels)):
            _check_tensor(t, self.src_dtype, n, f"source {i}")
            if t.device != dst.device:
                raise RuntimeError("sources and destination must be on one device.")
            self._src_array[i] = t.data_ptr()
        stream = torch.cuda.current_stream(dst.device).cuda_stream
        with torch.cuda.device(dst.device):
            _lib.check(
                _lib.lib().mfsdp_segment_program_run(self._handle, self._src_array, len(self.src_numels), dst.data_ptr(), stream)
            )
        return dst

    def run_many(self, srcs_per_buffer: Sequence[Sequence[torch.Tensor]], dsts: Sequence[torch.Tensor]) -> None:
        """The program over several buffers of this layout in one grid
        (``mfsdp_segment_program_run_many``): buffer ``b`` reads
        ``srcs_per_buffer[b]`` and writes ``dsts[b]``."""
        if self._handle is None:
            raise RuntimeError("segment program was destroyed.")
        if len(srcs_per_buffer) != len(dsts):
            raise RuntimeError(f"{len(srcs_per_buffer)} source lists for {len(dsts)} destinations.")
        if not dsts:
            return
        n_srcs = len(self.src_numels)
        src_array = (ctypes.c_void_p * max(1, n_srcs * len(dsts)))()
        dst_array = (ctypes.c_void_p * len(dsts))()
        device = dsts[0].device
        for b, (srcs, dst) in enumerate(zip(srcs_per_buffer, dsts)):
            if len(srcs) != n_srcs:
                raise RuntimeError(f"segment program expects {n_srcs} sources, got {len(srcs)} (buffer {b}).")
            _check_tensor(dst, self.dst_dtype, self.dst_numel, f"destination {b}")
            if dst.device != device:
                raise RuntimeError("every buffer of a batch must be on one device.")
            dst_array[b] = dst.data_ptr()
            for i, (t, n) in enumerate(zip(srcs, self.src_numels)):
                _check_tensor(t, self.src_dtype, n, f"source {i} of buffer {b}")
                if t.device != device:
                    raise RuntimeError("sources and destination must be on one device.")
                src_array[b * n_srcs + i] = t.data_ptr()
        stream = torch.cuda.current_stream(device).cuda_stream
        with torch.cuda.device(device):
            _lib.check(_lib.lib().mfsdp_segment_program_run_many(self._handle, len(dsts), src_array, n_srcs, dst_array, stream))

    def destroy(self) -> None:
        if getattr(self, "_handle", None) is not None:
            _lib.lib().mfsdp_segment_program_destroy(self._handle)
            self._handle = None

    def __del__(self) -> None:  # tables are small; freeing needs the library to be alive
        try:
            self.destroy()
        except Exception:
            pass


def _check_tensor(t: torch.Tensor, dtype: torch.dtype, min_numel: int, what: str) -> None:
    """The preconditions the reference checks before its copy kernels
    (matrix_fsdp/kernels/native.py:353-360, kernels/native/matrix_copy.cpp:60-78)."""
    if not t.is_cuda:
        raise RuntimeError(f"{what} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{what} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"{what} dtype mismatch: expected {dtype}, got {t.dtype}")
    if t.numel() < min_numel:
        raise RuntimeError(f"{what} has {t.numel()} elements, the layout needs {min_numel}")


# --------------------------------------------------------------------------- builders


def _segment_arrays(plan, *, padded: bool):
    """(global_start, shard-side offset, numel) of every segment of every rank;
    the shard-side offset is into the padded ``[W*max_shard]`` buffer or the
    compact rank-major one."""
    max_shard = max(plan.shard_sizes, default=0)
    gs, ls, ln = [], [], []
    base = 0
    for rank, segments in enumerate(plan.rank_segments):
        rank_base = rank * max_shard if padded else base
        for seg in segments:
            gs.append(seg.global_start)
            ls.append(rank_base + seg.local_start)
            ln.append(seg.global_end - seg.global_start)
        base += plan.shard_sizes[rank]
    return np.asarray(gs, dtype=np.int64), np.asarray(ls, dtype=np.int64), np.asarray(ln, dtype=np.int64)


def pack_program(plan, dtype: torch.dtype, *, padded: bool = True, out_dtype: torch.dtype | None = None, device="cuda") -> SegmentProgram:
    """full flat buffer -> every rank's shard.  ``padded`` writes the gathered
    all-gather layout ``[W*max_shard]`` with zeroed pad tails, otherwise the
    compact rank-major ``[sum shard_sizes]``.  ``out_dtype`` folds the
    param-dtype cast of the all-gather input (runtime/flat_buffer.py:309)."""
    gs, ls, ln = _segment_arrays(plan, padded=padded)
    dst_numel = len(plan.shard_sizes) * max(plan.shard_sizes, default=0) if padded else sum(plan.shard_sizes)
    runs = make_runs(gs, ls, ln)
    fills = fill_runs_for_gaps(runs, dst_numel)
    return SegmentProgram(np.concatenate((runs, fills)), (plan.total_numel,), dst_numel, src_dtype=dtype, dst_dtype=out_dtype, device=device)


def unpack_program(plan, dtype: torch.dtype, *, padded: bool = True, out_dtype: torch.dtype | None = None, device="cuda") -> SegmentProgram:
    """gathered shards (padded or compact) -> full flat buffer."""
    gs, ls, ln = _segment_arrays(plan, padded=padded)
    src_numel = len(plan.shard_sizes) * max(plan.shard_sizes, default=0) if padded else sum(plan.shard_sizes)
    return SegmentProgram(make_runs(ls, gs, ln), (src_numel,), plan.total_numel, src_dtype=dtype, dst_dtype=out_dtype, device=device)


def local_segments_program(segments, local_numel: int, output_numel: int, dtype: torch.dtype, device="cuda") -> SegmentProgram:
    """one rank's shard -> its slots of the full buffer."""
    gs = [s.global_start for s in segments]
    ls = [s.local_start for s in segments]
    ln = [s.global_end - s.global_start for s in segments]
    return SegmentProgram(make_runs(ls, gs, ln), (local_numel,), output_numel, src_dtype=dtype, device=device)


def take_local_segments_program(segments, full_numel: int, local_numel: int, dtype: torch.dtype, *, out_dtype: torch.dtype | None = None, device="cuda") -> SegmentProgram:
    """full flat buffer -> one rank's shard: the rank's row of ``pack_program``
    on its own, as a checkpoint load into another layout needs it
    (matrix_fsdp/checkpoint/state_dict.py:1330-1345)."""
    gs = [s.global_start for s in segments]
    ls = [s.local_start for s in segments]
    ln = [s.global_end - s.global_start for s in segments]
    return SegmentProgram(make_runs(gs, ls, ln), (full_numel,), local_numel, src_dtype=dtype, dst_dtype=out_dtype, device=device)


def grad_fill_runs(params, rank_segments, max_shard: int) -> np.ndarray:
    """Runs of the generic copy-in: for every (rank, segment ∩ parameter) the
    slice of that parameter's grad goes to ``[rank, local_start + ...]`` of the
    padded rank-major workspace (runtime/grad_bucket.py:209-225).  Source ``i``
    is parameter ``i``'s grad."""
    p_off = np.asarray([p.offset for p in params], dtype=np.int64)
    p_end = np.asarray([p.end for p in params], dtype=np.int64)
    order = np.argsort(p_off, kind="stable")
    so, se = p_off[order], p_end[order]
    src_off, dst_off, length, src_id = [], [], [], []
    for rank, segments in enumerate(rank_segments):
        if not segments:
            continue
        g0 = np.asarray([s.global_start for s in segments], dtype=np.int64)
        g1 = np.asarray([s.global_end for s in segments], dtype=np.int64)
        l0 = np.asarray([s.local_start for s in segments], dtype=np.int64)
        # parameters overlapping each segment form a contiguous range of the offset-sorted list
        first = np.searchsorted(se, g0, side="right")
        last = np.searchsorted(so, g1, side="left")
        for k in range(int((last - first).max(initial=0))):
            idx = first + k
            live = idx < last
            if not live.any():
                break
            pi = idx[live]
            a = np.maximum(so[pi], g0[live])
            b = np.minimum(se[pi], g1[live])
            ok = b > a
            src_off.append((a - so[pi])[ok])
            dst_off.append((rank * max_shard + l0[live] + a - g0[live])[ok])
            length.append((b - a)[ok])
            src_id.append(order[pi][ok])
    if not src_off:
        return np.zeros(0, dtype=RUN_DTYPE)
    runs = make_runs(np.concatenate(src_off), np.concatenate(dst_off), np.concatenate(length))
    runs["src_id"] = np.concatenate(src_id).astype(np.int32)
    # keep each source's runs together and in destination order so that neighbours can merge
    return runs[np.lexsort((runs["dst_off"], runs["src_id"]))]


def grad_fill_program(params, shard_sizes, rank_segments, grad_dtype: torch.dtype, reduce_dtype: torch.dtype | None = None, device="cuda") -> SegmentProgram:
    """per-parameter grads (separate allocations) -> ``packed [W*max_shard]``
    in the reduce dtype, pad tails zeroed: chunk-cat, flat-cat and the generic
    segment copy-in are all this one program (they differ only in layout)."""
    max_shard = max(shard_sizes, default=0)
    dst_numel = len(shard_sizes) * max_shard
    runs = grad_fill_runs(params, rank_segments, max_shard)
    fills = fill_runs_for_gaps(runs, dst_numel)
    return SegmentProgram(
        np.concatenate((runs, fills)), [p.numel for p in params], dst_numel, src_dtype=grad_dtype, dst_dtype=reduce_dtype, device=device
    )


def compact_owner_program(params, offsets: Sequence[int], total_numel: int, grad_dtype: torch.dtype, reduce_dtype: torch.dtype | None = None, device="cuda") -> SegmentProgram:
    """whole-parameter grads -> compact owner rank chunks ``[sum shard_sizes]``
    at the given packed offsets, everything else zero."""
    runs = make_runs(np.zeros(len(params), dtype=np.int64), np.asarray(offsets, dtype=np.int64), [p.numel for p in params])
    runs["src_id"] = np.arange(len(params), dtype=np.int32)
    fills = fill_runs_for_gaps(runs, total_numel)
    return SegmentProgram(
        np.concatenate((runs, fills)), [p.numel for p in params], total_numel, src_dtype=grad_dtype, dst_dtype=reduce_dtype, device=device
    )
