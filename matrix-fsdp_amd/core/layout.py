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


# ---------------------------------------------------------------------------
# Per-parameter view of a plan: what checkpoint metadata records.


@dataclass(frozen=True)
class ParamSegment:
    """The part of parameter ``fqn`` inside one of rank ``rank``'s segments;
    offsets as in ``LayoutSegment`` (matrix_fsdp/core/layout.py:33-55)."""

    fqn: str
    rank: int
    global_start: int
    global_end: int
    local_start: int

    @property
    def numel(self) -> int:
        return self.global_end - self.global_start

    @property
    def local_end(self) -> int:
        return self.local_start + self.numel

    def to_layout_segment(self) -> LayoutSegment:
        return LayoutSegment(self.global_start, self.global_end, self.local_start)


@dataclass(frozen=True)
class RankLayout:
    rank: int
    local_units: int
    segments: tuple[LayoutSegment, ...]


@dataclass(frozen=True)
class ParamLayout:
    fqn: str
    global_start: int
    global_end: int
    segments: tuple[ParamSegment, ...]

    @property
    def numel(self) -> int:
        return self.global_end - self.global_start


@dataclass(frozen=True)
class MatrixGroupLayout:
    """One unit's plan with the parameters cut along it
    (matrix_fsdp/core/layout.py:100-211).  Offsets are flat-buffer offsets of
    the unit, not of the model."""

    total_numel: int
    ranks: tuple[RankLayout, ...]
    params: tuple[ParamLayout, ...] = ()

    @classmethod
    def from_rank_segments(cls, total_numel: int, rank_segments: RankSegments, params: tuple[ParamLayout, ...] = ()) -> "MatrixGroupLayout":
        ranks = tuple(RankLayout(r, sum(s.numel for s in segs), tuple(segs)) for r, segs in enumerate(rank_segments))
        return cls(total_numel, ranks, tuple(params))

    @classmethod
    def from_shard_plan(cls, plan: ShardPlan, params: Sequence = ()) -> "MatrixGroupLayout":
        """``params`` are objects with ``fqn`` / ``offset`` / ``end``.  A
        parameter's segments are listed rank by rank, and inside a rank in the
        rank's segment order."""
        param_layouts = []
        for p in params:
            pieces = []
            for rank, segs in enumerate(plan.rank_segments):
                for seg in segs:
                    start, end = max(p.offset, seg.global_start), min(p.end, seg.global_end)
                    if start < end:
                        pieces.append(ParamSegment(p.fqn, rank, start, end, seg.local_start + start - seg.global_start))
            param_layouts.append(ParamLayout(p.fqn, p.offset, p.end, tuple(pieces)))
        return cls.from_rank_segments(plan.total_numel, plan.rank_segments, tuple(param_layouts))

    @property
    def world_size(self) -> int:
        return len(self.ranks)

    @property
    def shard_sizes(self) -> tuple[int, ...]:
        return tuple(rank.local_units for rank in self.ranks)

    @property
    def rank_segments(self) -> RankSegments:
        return tuple(rank.segments for rank in self.ranks)

    def param(self, fqn: str) -> ParamLayout:
        for layout in self.params:
            if layout.fqn == fqn:
                return layout
        raise KeyError(fqn)

    def owner_ranks(self, fqn: str) -> tuple[int, ...]:
        return tuple(sorted({seg.rank for seg in self.param(fqn).segments}))

    def rank_segments_for_param(self, rank: int, fqn: str) -> tuple[ParamSegment, ...]:
        return tuple(seg for seg in self.param(fqn).segments if seg.rank == rank)

    def params_for_rank(self, rank: int) -> tuple[str, ...]:
        return tuple(dict.fromkeys(seg.fqn for p in self.params for seg in p.segments if seg.rank == rank))

    def to_shard_plan(self) -> ShardPlan:
        return ShardPlan.from_rank_segments(self.total_numel, self.rank_segments)
