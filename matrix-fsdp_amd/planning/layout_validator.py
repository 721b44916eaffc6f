"""Checks a ``MatrixGroupLayout`` against the parameters it was planned for, and
says in which way a unit could run it.

``validate_group_layout`` (matrix_fsdp/planning/layout_validator.py:21-30) raises
``ValueError`` unless: the layout covers the managed parameters in their order
for the right number of ranks; every rank's segments are back to back in its
shard and all ranks' segments tile the flat buffer once; every parameter's
segments tile the parameter, stay inside it and inside their rank's shard, and
sit where the rank's segments put them; and the shard hints hold (whole
parameters unsplit, block / row-block cuts aligned, an expert group on one rank).

``explain_runtime_layout_compatibility`` (:33-88) names the execution mode:
``matrix_shard`` (one rank-ordered stretch per rank), ``segment_runtime``
(parameters split, but each rank holds at most one piece of a parameter and
nothing else shares that piece's segment), ``flat_reorder`` (whole parameters
in an order the flat buffer can adopt), else ``unsupported``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Sequence

from ..core.layout import LayoutSegment, MatrixGroupLayout
from ..core.managed_param import ParamRuntimeKind
from ..core.placement import explain_matrix_shard_compatibility


@dataclass(frozen=True)
class RuntimeLayoutCompatibility:
    compatible: bool
    mode: str
    reason: str | None = None
    requires_flat_reorder: bool = False
    matrix_shard_compatible: bool = False
    matrix_shard_reason: str | None = None


def _check_range(start: int, end: int, total: int, what: str) -> None:
    if start < 0 or end < 0 or start >= end or end > total:
        raise ValueError(f"Invalid {what} segment range [{start}, {end}) for total_numel={total}.")


def _check_tiling(pieces: Iterable[tuple[int, int, str]], start: int, end: int, what: str) -> None:
    """``pieces`` = (start, end, label); together they must cover [start, end) once."""
    cursor = start
    for lo, hi, label in sorted(pieces, key=lambda piece: piece[:2]):
        if lo < cursor:
            raise ValueError(f"{what} overlap at {label}; expected next start >= {cursor}.")
        if lo > cursor:
            raise ValueError(f"{what} gap before {label}; expected next start {cursor}.")
        cursor = hi
    if cursor != end:
        raise ValueError(f"{what} coverage ends at {cursor}, expected {end}.")


def _params_touching(segment: LayoutSegment, params: Sequence) -> list[str]:
    return [p.fqn for p in params if max(p.offset, segment.global_start) < min(p.end, segment.global_end)]


def validate_group_layout(layout: MatrixGroupLayout, params: Sequence, world_size: int) -> None:
    total = sum(p.numel for p in params)
    if layout.total_numel != total:
        raise ValueError(f"Group layout total_numel={layout.total_numel}, expected {total}.")
    if layout.world_size != world_size:
        raise ValueError(f"Group layout has {layout.world_size} ranks, expected world_size={world_size}.")
    have, want = tuple(p.fqn for p in layout.params), tuple(p.fqn for p in params)
    if have != want:
        raise ValueError(f"Group layout params {have} do not match managed params {want}.")

    # ranks: segments back to back in the shard, all of them tiling the flat buffer
    everything = []
    for rank, rank_layout in enumerate(layout.ranks):
        if rank_layout.rank != rank:
            raise ValueError(f"Rank layout at index {rank} has rank={rank_layout.rank}.")
        held = sum(seg.numel for seg in rank_layout.segments)
        if rank_layout.local_units != held:
            raise ValueError(f"Rank {rank} local_units={rank_layout.local_units}, expected {held} from segments.")
        cursor = 0
        for seg in rank_layout.segments:
            _check_range(seg.global_start, seg.global_end, layout.total_numel, f"rank {rank}")
            if seg.local_start != cursor:
                raise ValueError(f"Rank {rank} segment {seg} has local_start={seg.local_start}, expected contiguous local_start={cursor}.")
            cursor = seg.local_start + seg.numel
            everything.append((seg.global_start, seg.global_end, f"rank segment {seg}"))
    _check_tiling(everything, 0, layout.total_numel, "rank segments")

    # parameters: pieces tile the parameter and sit where the rank's segments say
    by_name = {p.fqn: p for p in params}
    for param_layout in layout.params:
        managed = by_name[param_layout.fqn]
        if (param_layout.global_start, param_layout.global_end) != (managed.offset, managed.end):
            raise ValueError(
                f"Param layout {param_layout.fqn} range [{param_layout.global_start}, {param_layout.global_end}) "
                f"does not match managed range [{managed.offset}, {managed.end})."
            )
        pieces = []
        for piece in param_layout.segments:
            if piece.fqn != param_layout.fqn:
                raise ValueError(f"Param {param_layout.fqn} contains segment for {piece.fqn}.")
            if not 0 <= piece.rank < layout.world_size:
                raise ValueError(f"Param {param_layout.fqn} segment has invalid rank={piece.rank}.")
            _check_range(piece.global_start, piece.global_end, layout.total_numel, f"param {param_layout.fqn}")
            if piece.global_start < managed.offset or piece.global_end > managed.end:
                raise ValueError(f"Param {param_layout.fqn} segment {piece} crosses parameter boundary.")
            if piece.local_start < 0 or piece.local_end > layout.ranks[piece.rank].local_units:
                raise ValueError(f"Param {param_layout.fqn} segment {piece} is outside rank {piece.rank} local shard.")
            pieces.append((piece.global_start, piece.global_end, f"param segment {piece}"))
        _check_tiling(pieces, managed.offset, managed.end, f"param {param_layout.fqn}")
    for param_layout in layout.params:
        for piece in param_layout.segments:
            placed = any(
                seg.global_start <= piece.global_start
                and piece.global_end <= seg.global_end
                and piece.local_start == seg.local_start + piece.global_start - seg.global_start
                for seg in layout.ranks[piece.rank].segments
            )
            if not placed:
                raise ValueError(f"Param {param_layout.fqn} segment {piece} does not project onto rank {piece.rank} segments.")

    # shard hints
    expert_ranks: dict[str, set[int]] = {}
    for managed, param_layout in zip(params, layout.params):
        hint = managed.shard_hint
        pieces = param_layout.segments
        if hint.split_granularity in ("parameter", "matrix_owner") and len(pieces) != 1:
            raise ValueError(f"Param {managed.fqn} split_granularity={hint.split_granularity!r} requires a single whole-parameter owner segment.")
        unit = None
        if hint.block_shape is not None and hint.split_granularity == "block":
            unit = hint.block_shape[0]
        if hint.block_shape is not None and hint.split_granularity == "row_block":
            unit = hint.block_shape[0] * tuple(managed.shape)[1]
        if unit is not None:
            for piece in pieces:
                if (piece.global_start - managed.offset) % unit or (piece.global_end - managed.offset) % unit:
                    raise ValueError(f"Param {managed.fqn} segment {piece} is not aligned to block_units={unit}.")
        if hint.runtime_kind == ParamRuntimeKind.EXPERT_OWNER:
            if len(pieces) != 1:
                raise ValueError(f"Param {managed.fqn} runtime_kind='expert_owner' requires one whole owner segment.")
            expert_ranks.setdefault(hint.expert_group_id or managed.fqn, set()).add(pieces[0].rank)
    for group, ranks in expert_ranks.items():
        if len(ranks) != 1:
            raise ValueError(f"Expert group {group!r} must have one owner rank, got {tuple(sorted(ranks))}.")


def _one_piece_per_param_and_rank(layout: MatrixGroupLayout, params: Sequence) -> str | None:
    """``None`` when every rank segment lies in exactly one parameter and no rank
    holds two segments of the same parameter; else what is wrong."""
    for rank, rank_layout in enumerate(layout.ranks):
        seen: set[str] = set()
        for seg in rank_layout.segments:
            touching = _params_touching(seg, params)
            if len(touching) != 1:
                return f"rank {rank} segment {seg} overlaps {len(touching)} parameters"
            if touching[0] in seen:
                return f"rank {rank} owns multiple local segments of parameter {touching[0]!r}"
            seen.add(touching[0])
    return None


def explain_runtime_layout_compatibility(
    layout: MatrixGroupLayout,
    params: Sequence,
    world_size: int,
    *,
    allow_flat_reorder: bool = True,
    allow_segment_runtime: bool = True,
) -> RuntimeLayoutCompatibility:
    validate_group_layout(layout, params, world_size)
    placement = explain_matrix_shard_compatibility(layout)
    if placement.compatible:
        return RuntimeLayoutCompatibility(True, "matrix_shard", matrix_shard_compatible=True)

    split = any(len(p.segments) > 1 for p in layout.params)
    per_piece_problem = _one_piece_per_param_and_rank(layout, params)
    if split and sum(layout.shard_sizes) == layout.total_numel and per_piece_problem is None:
        if not allow_segment_runtime:
            return RuntimeLayoutCompatibility(
                False, "unsupported", "layout requires segment_runtime, but segment runtime layouts are disabled", matrix_shard_reason=placement.reason
            )
        return RuntimeLayoutCompatibility(True, "segment_runtime", placement.reason, matrix_shard_reason=placement.reason)

    by_name = {p.fqn: p for p in params}
    whole = all(
        len(p.segments) == 1 and (p.segments[0].global_start, p.segments[0].global_end) == (by_name[p.fqn].offset, by_name[p.fqn].end)
        for p in layout.params
    )
    if allow_flat_reorder and placement.requires_flat_reorder and whole:
        return RuntimeLayoutCompatibility(True, "flat_reorder", placement.reason, requires_flat_reorder=True, matrix_shard_reason=placement.reason)

    reason = per_piece_problem
    if reason is None and split:
        name = next(p.fqn for p in layout.params if len(p.segments) > 1)
        reason = f"parameter {name!r} is split in a layout that cannot be exposed as local views"
    return RuntimeLayoutCompatibility(
        False,
        "unsupported",
        reason or placement.reason or "layout is not rank-contiguous and cannot be flat-reordered",
        requires_flat_reorder=placement.requires_flat_reorder,
        matrix_shard_reason=placement.reason,
    )


def validate_runtime_layout(
    layout: MatrixGroupLayout,
    params: Sequence,
    world_size: int,
    *,
    allow_flat_reorder: bool = True,
    allow_segment_runtime: bool = True,
) -> RuntimeLayoutCompatibility:
    verdict = explain_runtime_layout_compatibility(
        layout, params, world_size, allow_flat_reorder=allow_flat_reorder, allow_segment_runtime=allow_segment_runtime
    )
    if not verdict.compatible:
        raise ValueError(f"MatrixFSDP runtime cannot execute planner layout. Reason: {verdict.reason}.")
    return verdict
