"""Whole-parameter owner layouts: every parameter lives whole on one rank.

These are the layouts the Muon path needs (the update orthogonalises whole
matrices, so a matrix must not be cut): the reference's
``ordered_matrix_owner_tail_plan`` (matrix_fsdp/planning/planner.py:129-156),
``load_balanced_matrix_owner_tail_plan`` (:159-207) and its multi-group form
(:210-271).  A *role* is one 2-D parameter, or all the non-2-D parameters of
a group together (the tail); roles go to ranks, largest first, and each rank's
shard is its parameters back to back in the order they were assigned
(:342-387).  The functions return ``ShardPlan`` s.
"""
from __future__ import annotations

from typing import Sequence

from ..core.layout import LayoutSegment, ShardPlan


def _check_world(world_size: int) -> None:
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, got {world_size}.")


def _merge_adjacent(segments: Sequence[LayoutSegment]) -> tuple[LayoutSegment, ...]:
    """Neighbouring segments that continue each other both in the flat buffer
    and in the shard become one (planner.py:390-407)."""
    merged: list[LayoutSegment] = []
    for seg in segments:
        if merged and merged[-1].global_end == seg.global_start and merged[-1].local_start + merged[-1].numel == seg.local_start:
            merged[-1] = LayoutSegment(merged[-1].global_start, seg.global_end, merged[-1].local_start)
        else:
            merged.append(seg)
    return tuple(merged)


def whole_param_assignment_plan(params: Sequence, world_size: int, assignments: Sequence[tuple[object, int]], *, merge_adjacent_rank_segments: bool = False) -> ShardPlan:
    """``assignments`` lists ``(param, rank)`` in the order the parameters are
    laid out inside their rank's shard."""
    _check_world(world_size)
    segments: list[list[LayoutSegment]] = [[] for _ in range(world_size)]
    sizes = [0] * world_size
    for param, rank in assignments:
        if not 0 <= rank < world_size:
            raise ValueError(f"Owner rank for parameter {param.fqn!r} must be in [0, {world_size}), got {rank}.")
        segments[rank].append(LayoutSegment(param.offset, param.end, sizes[rank]))
        sizes[rank] += param.numel
    if len(assignments) != len(params):
        raise ValueError("every parameter needs exactly one owner.")
    planned = [_merge_adjacent(s) if merge_adjacent_rank_segments else tuple(s) for s in segments]
    return ShardPlan.from_rank_segments(sum(p.numel for p in params), planned)


def owner_ranks(plan: ShardPlan, param) -> tuple[int, ...]:
    """Ranks whose shard holds any part of ``param``."""
    return tuple(
        rank
        for rank, segments in enumerate(plan.rank_segments)
        if any(seg.global_start < param.end and param.offset < seg.global_end for seg in segments)
    )


def _split_roles(params: Sequence) -> tuple[list, list]:
    return [p for p in params if len(p.shape) == 2], [p for p in params if len(p.shape) != 2]


def ordered_matrix_owner_tail_plan(params: Sequence, world_size: int) -> ShardPlan:
    """Matrices to ranks 0, 1, 2, ... in module order (wrapping around), the
    tail to the rank after the last matrix owner, or to the last rank when the
    matrices already use them all."""
    _check_world(world_size)
    matrices, tail = _split_roles(params)
    tail_rank = min(len(matrices), world_size - 1)
    assignments = [(p, i % world_size) for i, p in enumerate(matrices)] + [(p, tail_rank) for p in tail]
    return whole_param_assignment_plan(params, world_size, assignments)


def _initial_units(initial_rank_units: Sequence[int] | None, world_size: int) -> list[int]:
    if initial_rank_units is None:
        return [0] * world_size
    if len(initial_rank_units) != world_size:
        raise ValueError(f"initial_rank_units length must match world_size={world_size}, got {len(initial_rank_units)}.")
    return list(initial_rank_units)


def _fixed_owner(role_params: Sequence, world_size: int) -> int | None:
    """An ``owner_rank`` hint pins a role (planner.py:410-425)."""
    wanted = {getattr(getattr(p, "shard_hint", None), "owner_rank", None) for p in role_params} - {None}
    if not wanted:
        return None
    if len(wanted) != 1:
        raise ValueError(f"Conflicting owner_rank hints for params: {', '.join(p.fqn for p in role_params)}.")
    rank = wanted.pop()
    if rank >= world_size:
        raise ValueError(f"owner_rank={rank} must be in [0, {world_size}).")
    return rank


def _lightest(units: Sequence[int]) -> int:
    return min(range(len(units)), key=lambda r: (units[r], r))


def load_balanced_matrix_owner_tail_plan(
    params: Sequence, world_size: int, *, initial_rank_units: Sequence[int] | None = None, merge_adjacent_rank_segments: bool = False
) -> ShardPlan:
    """Roles, largest first (ties in module order), each to the rank that is
    lightest at that moment (ties to the lower rank)."""
    return load_balanced_matrix_owner_tail_group_plans(
        (params,), world_size, initial_rank_units=initial_rank_units, merge_adjacent_rank_segments=merge_adjacent_rank_segments, honour_owner_hints=False
    )[0]


def load_balanced_matrix_owner_tail_group_plans(
    param_groups: Sequence[Sequence],
    world_size: int,
    *,
    initial_rank_units: Sequence[int] | None = None,
    merge_adjacent_rank_segments: bool = True,
    honour_owner_hints: bool = True,
    rank_units_out: list[int] | None = None,
) -> tuple[ShardPlan, ...]:
    """One plan per group, the owners decided over the roles of *all* groups
    at once (largest first, then group order, then module order), so that the
    ranks end up evenly loaded across the whole model rather than per group.
    ``rank_units_out`` receives the final load per rank."""
    _check_world(world_size)
    units = _initial_units(initial_rank_units, world_size)
    roles = []
    for g, params in enumerate(param_groups):
        matrices, tail = _split_roles(params)
        roles.extend((p.numel, g, i, (p,)) for i, p in enumerate(matrices))
        if tail:
            roles.append((sum(p.numel for p in tail), g, len(matrices), tuple(tail)))
    assignments: list[list[tuple[object, int]]] = [[] for _ in param_groups]
    for numel, g, _, role_params in sorted(roles, key=lambda role: (-role[0], role[1], role[2])):
        rank = _fixed_owner(role_params, world_size) if honour_owner_hints else None
        if rank is None:
            rank = _lightest(units)
        assignments[g].extend((p, rank) for p in role_params)
        units[rank] += numel
    if rank_units_out is not None:
        rank_units_out[:] = units
    return tuple(
        whole_param_assignment_plan(params, world_size, assignments[g], merge_adjacent_rank_segments=merge_adjacent_rank_segments)
        for g, params in enumerate(param_groups)
    )


class MuonOwnerPlanner:
    """Planner for ``fully_shard(..., optimizer_policy="muon")``: called once per
    unit, it keeps the load every rank has been given so far and places each
    new unit's roles on the lightest ranks ("role greedy", the owner assignment
    the reference pairs with its Muon policies, matrix_fsdp/api.py:186-187)."""

    def __init__(self) -> None:
        self.rank_units: list[int] | None = None

    def __call__(self, params: Sequence, world_size: int) -> ShardPlan:
        if self.rank_units is None or len(self.rank_units) != world_size:
            self.rank_units = [0] * world_size
        out: list[int] = []
        plan = load_balanced_matrix_owner_tail_group_plans(
            (params,), world_size, initial_rank_units=self.rank_units, merge_adjacent_rank_segments=False, rank_units_out=out
        )[0]
        self.rank_units = out
        return plan
