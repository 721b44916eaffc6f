"""Segment coalescing (matrix_fsdp/kernels/segment_fusion.py:6-29)."""
from __future__ import annotations

from ..core.layout import LayoutSegment


def coalesce_contiguous_segments(segments: tuple[LayoutSegment, ...]) -> tuple[LayoutSegment, ...]:
    """Neighbours that continue each other both in the flat buffer and in the
    local shard become one segment; gaps on either side are preserved."""
    fused: list[LayoutSegment] = []
    for seg in segments:
        if fused and fused[-1].global_end == seg.global_start and fused[-1].local_end == seg.local_start:
            fused[-1] = LayoutSegment(fused[-1].global_start, seg.global_end, fused[-1].local_start)
        else:
            fused.append(seg)
    return tuple(fused)


def coalesce_rank_segments(rank_segments):
    return tuple(coalesce_contiguous_segments(segments) for segments in rank_segments)
