"""Geometry of the padded rank-chunk buffers a shard plan implies.

One descriptor stands in for the reference's ``StaticParamBufferLayout``
(matrix_fsdp/runtime/static_param_buffer.py:9-88) and
``ElasticParamBufferLayout`` (runtime/elastic_param_buffer.py:111-214), which
share these properties; only the arithmetic is kept (no caches or pools).
"""
from __future__ import annotations

from dataclasses import dataclass

from ..core.layout import LayoutSegment, ShardPlan

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
