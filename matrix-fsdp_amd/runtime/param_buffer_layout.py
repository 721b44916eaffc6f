"""Geometry of the padded rank-chunk buffers a shard plan implies.

One descriptor stands in for the reference's ``StaticParamBufferLayout``
(matrix_fsdp/runtime/static_param_buffer.py:9-88) and
``ElasticParamBufferLayout`` (runtime/elastic_param_buffer.py:111-214), which
share these properties (both names are bound to it); only the arithmetic is
kept (no caches or pools).  ``build_communication_plan`` precomputes what an
exchange of the layout's shards walks over: the segments, the same with
neighbours merged, one chunk per segment, and the rank-chunk sizes when every
rank holds a single stretch (elastic_param_buffer.py:17-81, 197-214).
"""
from __future__ import annotations

from dataclasses import dataclass

from ..core.layout import LayoutSegment, ShardPlan
from ..kernels.segment_fusion import coalesce_rank_segments

RankSegments = tuple[tuple[LayoutSegment, ...], ...]


def rank_chunk_shard_sizes(rank_segments: RankSegments) -> tuple[int, ...] | None:
    """Shard sizes when every rank holds one contiguous chunk of the flat
    buffer in rank order (empty ranks allowed), else ``None``
    (matrix_fsdp/kernels/custom_collectives.py:1035-1051)."""
    cursor, sizes = 0, []
    for segments in rank_segments:
        if not segments:
            sizes.append(0)
            continue
        if len(segments) != 1:
            return None
        seg = segments[0]
        if seg.global_start != cursor or seg.local_start != 0:
            return None
        sizes.append(seg.numel)
        cursor = seg.global_end
    return tuple(sizes)


def rank_segments_are_rank_contiguous_chunks(rank_segments: RankSegments | None) -> bool:
    """runtime/static_param_buffer.py:192-207."""
    return rank_segments is not None and rank_chunk_shard_sizes(rank_segments) is not None


def packed_rank_shards_are_full_tensor_order(total_numel: int, shard_sizes, rank_segments: RankSegments | None) -> bool:
    """True when the compact rank-major concatenation of the shards already is
    the flat buffer, so unpack is the identity
    (runtime/flat_buffer.py:1335-1353, runtime/static_param_buffer.py:55-74)."""
    if total_numel != sum(shard_sizes):
        return False
    if rank_segments is None:
        return True
    base = 0
    for rank, segments in enumerate(rank_segments):
        cursor = 0
        for seg in segments:
            if seg.local_start != cursor or seg.global_start != base + cursor:
                return False
            cursor = seg.local_end
        if cursor != shard_sizes[rank]:
            return False
        base += shard_sizes[rank]
    return True


def rank_segments_from_shard_sizes(shard_sizes) -> RankSegments:
    """One stretch per non-empty rank, in rank order (elastic_param_buffer.py:506-515)."""
    cursor, out = 0, []
    for size in shard_sizes:
        out.append((LayoutSegment(cursor, cursor + size, 0),) if size else ())
        cursor += size
    return tuple(out)


@dataclass(frozen=True)
class ElasticRankChunk:
    rank: int
    global_start: int
    global_end: int
    local_start: int = 0

    @property
    def numel(self) -> int:
        return self.global_end - self.global_start

    def as_segment(self) -> LayoutSegment:
        return LayoutSegment(self.global_start, self.global_end, self.local_start)


@dataclass(frozen=True)
class ElasticCommunicationPlan:
    rank_segments: RankSegments
    coalesced_rank_segments: RankSegments
    rank_chunks: tuple[ElasticRankChunk, ...]
    rank_chunk_shard_sizes: tuple[int, ...] | None
    rank_chunk_segments: RankSegments | None
    rank_chunk_fast_path: bool
    packed_full_order: bool

    @property
    def world_size(self) -> int:
        return len(self.rank_segments)

    @property
    def segment_count(self) -> int:
        return sum(len(s) for s in self.rank_segments)

    @property
    def coalesced_segment_count(self) -> int:
        return sum(len(s) for s in self.coalesced_rank_segments)

    @property
    def max_segments_per_rank(self) -> int:
        return max((len(s) for s in self.rank_segments), default=0)

    @property
    def max_coalesced_segments_per_rank(self) -> int:
        return max((len(s) for s in self.coalesced_rank_segments), default=0)

    @property
    def rank_chunk_count(self) -> int:
        return len(self.rank_chunks)

    @property
    def nonempty_rank_chunk_count(self) -> int:
        return sum(1 for chunk in self.rank_chunks if chunk.numel > 0)

    def as_summary(self) -> dict[str, object]:
        return {
            "communication_plan_segment_count": self.segment_count,
            "communication_plan_coalesced_segment_count": self.coalesced_segment_count,
            "communication_plan_max_segments_per_rank": self.max_segments_per_rank,
            "communication_plan_max_coalesced_segments_per_rank": self.max_coalesced_segments_per_rank,
            "communication_plan_rank_chunk_count": self.rank_chunk_count,
            "communication_plan_nonempty_rank_chunk_count": self.nonempty_rank_chunk_count,
            "communication_plan_rank_chunk_fast_path": self.rank_chunk_fast_path,
            "communication_plan_packed_full_order": self.packed_full_order,
            "communication_plan_has_rank_chunk_shard_sizes": self.rank_chunk_shard_sizes is not None,
        }


@dataclass(frozen=True)
class ParamBufferLayout:
    total_numel: int
    shard_sizes: tuple[int, ...]
    rank_segments: RankSegments | None

    @classmethod
    def from_plan(cls, plan: ShardPlan) -> "ParamBufferLayout":
        return cls(plan.total_numel, tuple(plan.shard_sizes), plan.rank_segments)

    @property
    def world_size(self) -> int:
        return len(self.shard_sizes)

    @property
    def total_shard_numel(self) -> int:
        return sum(self.shard_sizes)

    @property
    def max_shard_size(self) -> int:
        return max(self.shard_sizes, default=0)

    @property
    def min_shard_size(self) -> int:
        return min(self.shard_sizes, default=0)

    @property
    def padded_numel(self) -> int:
        """Elements of the all-gather / reduce-scatter workspace: ``W * max_shard``."""
        return self.world_size * self.max_shard_size

    @property
    def padding_waste_numel(self) -> int:
        return max(self.padded_numel - self.total_shard_numel, 0)

    @property
    def padding_waste_ratio(self) -> float:
        return self.padding_waste_numel / self.total_shard_numel if self.total_shard_numel else 0.0

    @property
    def owner_imbalance_ratio(self) -> float:
        """Largest shard over the mean shard (runtime/elastic_param_buffer.py:146-148)."""
        mean = self.total_shard_numel / self.world_size if self.world_size else 0.0
        return self.max_shard_size / mean if mean else 0.0

    @property
    def segment_count(self) -> int:
        return sum(len(s) for s in self.rank_segments or ())

    @property
    def max_segments_per_rank(self) -> int:
        return max((len(s) for s in self.rank_segments or ()), default=0)

    @property
    def rank_chunk_fast_path(self) -> bool:
        return rank_segments_are_rank_contiguous_chunks(self.rank_segments)

    @property
    def packed_rank_shards_are_full_tensor_order(self) -> bool:
        return packed_rank_shards_are_full_tensor_order(self.total_numel, self.shard_sizes, self.rank_segments)

    def rank_chunk_workspace_numel(self, *, compact: bool) -> int:
        """Size of the gradient rank-chunk workspace: compact ``sum shard_sizes``
        or padded ``W * max_shard``."""
        return self.total_shard_numel if compact else self.padded_numel

    def build_communication_plan(self) -> ElasticCommunicationPlan:
        segments = self.rank_segments or rank_segments_from_shard_sizes(self.shard_sizes)
        chunk_sizes = rank_chunk_shard_sizes(segments)
        return ElasticCommunicationPlan(
            rank_segments=segments,
            coalesced_rank_segments=coalesce_rank_segments(segments),
            rank_chunks=tuple(ElasticRankChunk(rank, s.global_start, s.global_end, s.local_start) for rank, segs in enumerate(segments) for s in segs),
            rank_chunk_shard_sizes=chunk_sizes,
            rank_chunk_segments=None if chunk_sizes is None else rank_segments_from_shard_sizes(chunk_sizes),
            rank_chunk_fast_path=chunk_sizes is not None,
            packed_full_order=self.packed_rank_shards_are_full_tensor_order,
        )

    def as_summary(self) -> dict[str, object]:
        return {
            "rank_chunk_fast_path": self.rank_chunk_fast_path,
            "packed_rank_shards_are_full_tensor_order": self.packed_rank_shards_are_full_tensor_order,
            "segment_count": self.segment_count,
            "max_segments_per_rank": self.max_segments_per_rank,
            "shard_sizes": self.shard_sizes,
            "max_shard_size": self.max_shard_size,
            "min_shard_size": self.min_shard_size,
            "padding_waste_numel": self.padding_waste_numel,
            "padding_waste_ratio": self.padding_waste_ratio,
            "owner_imbalance_ratio": self.owner_imbalance_ratio,
        }


StaticParamBufferLayout = ParamBufferLayout
ElasticParamBufferLayout = ParamBufferLayout
