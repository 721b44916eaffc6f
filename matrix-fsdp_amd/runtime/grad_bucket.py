"""Gradient copy-in: per-parameter grads -> the rank-major reduce-scatter input.

Same surface as the reference's ``matrix_fsdp/runtime/grad_bucket.py``
(``MatrixGradBucket``, ``classify_copy_in_layout``,
``fill_reduce_scatter_input(bucket, packed, backend=...)``).  The reference
picks between ``torch.cat``, ``torch._foreach_copy_``, ``torch._chunk_cat`` and
a per-segment ``copy_`` loop (:97-116); here every backend is the same single
HIP launch -- a segment program compiled from the bucket's layout -- and the
backend name only selects which layouts are admissible, with the reference's
error messages.  The program also folds the grad -> reduce-dtype cast
(runtime/flat_buffer.py:612) and zeroes the pad tails (``packed.zero_()`` /
``_chunk_cat`` padding), so bf16 grads reach an fp32 workspace in one pass.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Literal

import torch

from ..core.layout import LayoutSegment
from ..core.managed_param import ManagedParam
from ..kernels.segment_program import SegmentProgram, grad_fill_program

CopyInBackend = Literal["auto", "flat_cat", "foreach_copy", "chunk_cat", "segment_copy"]
CopyInLayoutKind = Literal["flat_contiguous", "fsdp2_chunk", "generic_segment"]
_BACKENDS = ("auto", "flat_cat", "foreach_copy", "chunk_cat", "segment_copy")


@dataclass(frozen=True)
class BucketParamGrad:
    managed_param: ManagedParam
    grad: torch.Tensor


@dataclass(frozen=True)
class MatrixGradBucket:
    """matrix_fsdp/runtime/grad_bucket.py:21-40."""

    param_grads: tuple[BucketParamGrad, ...]
    total_numel: int
    shard_sizes: tuple[int, ...]
    rank_segments: tuple[tuple[LayoutSegment, ...], ...]
    packed_input: torch.Tensor | None = None
    packed_input_is_compact: bool = False

    @property
    def world_size(self) -> int:
        return len(self.shard_sizes)

    @property
    def max_shard_size(self) -> int:
        return max(self.shard_sizes, default=0)

    @property
    def has_grads(self) -> bool:
        return bool(self.param_grads) or self.packed_input is not None


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def _is_flat_contiguous(bucket: MatrixGradBucket) -> bool:
    """Equal shards, one segment per rank covering the buffer in rank order,
    parameters back to back (grad_bucket.py:127-155)."""
    if not bucket.param_grads or len(set(bucket.shard_sizes)) != 1:
        return False
    cursor = 0
    for size, segments in zip(bucket.shard_sizes, bucket.rank_segments):
        if len(segments) != 1:
            return False
        seg = segments[0]
        if seg.local_start != 0 or seg.global_start != cursor or seg.global_end != cursor + size:
            return False
        cursor = seg.global_end
    if cursor != bucket.total_numel:
        return False
    cursor = 0
    for pg in bucket.param_grads:
        mp = pg.managed_param
        if mp.offset != cursor or mp.end != cursor + mp.numel or pg.grad.numel() != mp.numel:
            return False
        cursor = mp.end
    return cursor == bucket.total_numel


def _is_fsdp2_chunk(bucket: MatrixGradBucket) -> bool:
    """Every parameter cut in ``W`` chunks of ``ceil(n/W)``, rank ``r`` storing
    chunk ``r`` of each in parameter order (grad_bucket.py:158-187)."""
    world = bucket.world_size
    if not bucket.param_grads or world == 0:
        return False
    table, cursor = [], 0
    for pg in bucket.param_grads:
        mp = pg.managed_param
        if pg.grad.numel() != mp.numel or mp.end != mp.offset + mp.numel:
            return False
        size = _ceil_div(mp.numel, world)
        table.append((mp, cursor, size))
        cursor += size
    if bucket.max_shard_size != cursor or any(s != cursor for s in bucket.shard_sizes):
        return False
    for rank in range(world):
        expected = []
        for mp, local_start, size in table:
            start = mp.offset + rank * size
            end = min(mp.end, start + size)
            if start < end:
                expected.append(LayoutSegment(start, end, local_start))
        if tuple(bucket.rank_segments[rank]) != tuple(expected):
            return False
    return True


def classify_copy_in_layout(bucket: MatrixGradBucket) -> CopyInLayoutKind:
    if _is_flat_contiguous(bucket):
        return "flat_contiguous"
    if _is_fsdp2_chunk(bucket):
        return "fsdp2_chunk"
    return "generic_segment"


@dataclass
class CopyInProgramCache:
    """Compiled copy-in programs of one flat buffer, keyed by the grad and
    workspace dtypes (the layout itself is fixed for the buffer's lifetime)."""

    programs: dict[tuple, SegmentProgram] = field(default_factory=dict)

    def get(self, bucket: MatrixGradBucket, grad_dtype: torch.dtype, packed_dtype: torch.dtype, device) -> SegmentProgram:
        key = (
            grad_dtype,
            packed_dtype,
            torch.device(device).index,
            tuple((pg.managed_param.offset, pg.managed_param.end) for pg in bucket.param_grads),
            bucket.shard_sizes,
            bucket.rank_segments,
        )
        program = self.programs.get(key)
        if program is None:
            params = [pg.managed_param for pg in bucket.param_grads]
            program = grad_fill_program(params, bucket.shard_sizes, bucket.rank_segments, grad_dtype, packed_dtype, device=device)
            self.programs[key] = program
        return program


_DEFAULT_CACHE = CopyInProgramCache()


def new_reduce_scatter_input(bucket: MatrixGradBucket, reference: torch.Tensor) -> torch.Tensor:
    if bucket.world_size == 0:
        raise ValueError("MatrixGradBucket requires at least one rank.")
    return reference.new_empty(bucket.world_size * bucket.max_shard_size)


def build_reduce_scatter_input(bucket: MatrixGradBucket, reference: torch.Tensor, *, backend: CopyInBackend = "auto") -> torch.Tensor:
    """``[rank0_padded_chunk, rank1_padded_chunk, ...]`` in ``reference``'s
    dtype and device (grad_bucket.py:43-62)."""
    if bucket.world_size == 0:
        raise ValueError("MatrixGradBucket requires at least one rank.")
    if bucket.packed_input is not None:
        return bucket.packed_input
    return fill_reduce_scatter_input(bucket, new_reduce_scatter_input(bucket, reference), backend=backend)


def fill_reduce_scatter_input(
    bucket: MatrixGradBucket,
    packed: torch.Tensor,
    *,
    backend: CopyInBackend = "auto",
    cache: CopyInProgramCache | None = None,
) -> torch.Tensor:
    """grad_bucket.py:71-116 as one HIP launch.  ``packed.dtype`` may differ
    from the grads' dtype for bfloat16 <-> float32 (the reduce-dtype cast)."""
    if bucket.world_size == 0:
        raise ValueError("MatrixGradBucket requires at least one rank.")
    expected = bucket.world_size * bucket.max_shard_size
    if packed.ndim != 1:
        raise ValueError(f"packed must be 1D, got shape {tuple(packed.shape)}.")
    if packed.numel() != expected:
        raise ValueError(f"packed has {packed.numel()} elements, expected {expected}.")
    if backend not in _BACKENDS:
        raise ValueError("backend must be 'auto', 'flat_cat', 'foreach_copy', 'chunk_cat', or 'segment_copy'.")
    kind = classify_copy_in_layout(bucket)
    if backend in ("flat_cat", "foreach_copy") and kind != "flat_contiguous":
        raise ValueError(f"{backend} backend requires an equal, rank-contiguous flat bucket layout.")
    if backend == "chunk_cat" and kind != "fsdp2_chunk":
        raise ValueError("chunk_cat backend requires an FSDP2-style per-parameter chunk bucket layout.")
    grads = []
    for pg in bucket.param_grads:
        grad = pg.grad.reshape(-1)
        if grad.numel() != pg.managed_param.numel:
            raise RuntimeError(f"Gradient for {pg.managed_param.fqn} has {grad.numel()} elements, expected {pg.managed_param.numel}.")
        grads.append(grad)
    if not grads:
        packed.zero_()
        return packed
    grad_dtype = grads[0].dtype
    if any(g.dtype != grad_dtype for g in grads):
        raise RuntimeError("all gradients of a bucket must share one dtype.")
    program = (cache or _DEFAULT_CACHE).get(bucket, grad_dtype, packed.dtype, packed.device)
    program.run(grads, packed)
    return packed
