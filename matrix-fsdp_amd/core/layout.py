"""Shard metadata for one flat parameter buffer.

A *flat buffer* is the concatenation of a unit's parameters in
``named_parameters`` order; every offset below counts elements of that
buffer.  A rank's *local shard* is the concatenation of its segments in
``local_start`` order.  Field names and meanings match the reference's
``LayoutSegment`` / ``ShardPlan`` (matrix_fsdp/core/layout.py:15-78) so that
plans produced by either side describe the same bytes.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Sequence


@dataclass(frozen=True)
class LayoutSegment:
    """``full[global_start:global_end]`` lives at ``local[local_start:...]``.

    Mirrors matrix_fsdp/core/layout.py:15-30.
    """

    global_start: int
    global_end: int
    local_start: int

    @property
    def numel(self) -> int:
        return self.global_end - self.global_start

    @property
    def local_end(self) -> int:
        return self.local_start + self.numel

    def intersects(self, start: int, end: int) -> bool:
        return max(self.global_start, start) < min(self.global_end, end)


RankSegments = tuple[tuple[LayoutSegment, ...], ...]


@dataclass(frozen=True)
class ShardPlan:
    """Which elements of the flat buffer each rank holds.

    Mirrors matrix_fsdp/core/layout.py:57-78: when ``rank_segments`` is not
    given every rank owns the single contiguous range
    ``[shard_offsets[r], shard_offsets[r] + shard_sizes[r])``.
    """

    total_numel: int
    shard_sizes: tuple[int, ...]
    shard_offsets: tuple[int, ...]
    rank_segments: RankSegments | None = None

    def __post_init__(self) -> None:
        if self.rank_segments is None:
            derived = tuple(
                (LayoutSegment(off, off + size, 0),)
                for off, size in zip(self.shard_offsets, self.shard_sizes)
            )
            object.__setattr__(self, "rank_segments", derived)

    @property
    def world_size(self) -> int:
        return len(self.shard_sizes)

    @property
    def max_shard_size(self) -> int:
        return max(self.shard_sizes, default=0)

    def local_range(self, rank: int) -> tuple[int, int]:
        start = self.shard_offsets[rank]
        return start, start + self.shard_sizes[rank]

    def local_segments(self, rank: int) -> tuple[LayoutSegment, ...]:
        return self.rank_segments[rank]

    def rank_packed_offset(self, rank: int) -> int:
        """Start of rank ``rank``'s shard in the compact rank-major order
        (matrix_fsdp/runtime/flat_buffer.py:1362-1363)."""
        return sum(self.shard_sizes[:rank])

    @classmethod
    def from_rank_segments(cls, total_numel: int, rank_segments: Iterable[Sequence[LayoutSegment]]) -> "ShardPlan":
        """Shard sizes are the per-rank segment totals and offsets their running
        sum, as ``MatrixGroupLayout.to_shard_plan`` builds them
        (matrix_fsdp/core/layout.py:191-203)."""
        segs = tuple(tuple(s) for s in rank_segments)
        sizes = tuple(sum(s.numel for s in rs) for rs in segs)
        offsets, cursor = [], 0
        for size in sizes:
            offsets.append(cursor)
            cursor += size
        return cls(total_numel, sizes, tuple(offsets), segs)


def validate_shard_plan(plan: ShardPlan) -> None:
    """Checks the invariants every copy entry point relies on: segments of a
    rank are laid out back to back in ``local_start`` order, fill exactly the
    rank's shard, stay inside the flat buffer and cover it exactly once."""
    if len(plan.shard_sizes) != len(plan.rank_segments):
        raise ValueError("rank_segments and shard_sizes disagree on the world size.")
    covered: list[tuple[int, int]] = []
    for rank, segments in enumerate(plan.rank_segments):
        cursor = 0
        for seg in segments:
            if seg.numel < 0 or seg.global_start < 0 or seg.global_end > plan.total_numel:
                raise ValueError(f"rank {rank}: segment {seg} leaves the flat buffer.")
            if seg.local_start != cursor:
                raise ValueError(f"rank {rank}: segment {seg} does not start at local offset {cursor}.")
            cursor = seg.local_end
            if seg.numel:
                covered.append((seg.global_start, seg.global_end))
        if cursor != plan.shard_sizes[rank]:
            raise ValueError(f"rank {rank}: segments hold {cursor} elements, shard size is {plan.shard_sizes[rank]}.")
    covered.sort()
    cursor = 0
    for start, end in covered:
        if start != cursor:
            raise ValueError(f"flat buffer range [{cursor}, {start}) is owned by {'no' if start > cursor else 'more than one'} rank.")
        cursor = end
    if cursor != plan.total_numel:
        raise ValueError(f"segments cover {cursor} of {plan.total_numel} elements.")
