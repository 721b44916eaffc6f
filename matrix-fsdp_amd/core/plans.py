"""Closed-form shard plans for the layouts the copy path is exercised on.

Each function takes the flat-buffer extents of the parameters (anything with
``offset`` / ``end`` / ``numel`` / ``shape``) and returns a ``ShardPlan``.
They restate, as closed forms, what the reference's planners emit for these
cases; they are not a planner.
"""
from __future__ import annotations

from typing import Sequence

from .layout import LayoutSegment, ShardPlan


def contiguous_even_plan(total_numel: int, world_size: int) -> ShardPlan:
    """Rank-contiguous even split of the flat buffer; the first
    ``total % W`` ranks hold one extra element
    (matrix_fsdp/planning/planner.py:46-56)."""
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, got {world_size}.")
    base, extra = divmod(total_numel, world_size)
    sizes = tuple(base + (r < extra) for r in range(world_size))
    offsets = tuple(sum(sizes[:r]) for r in range(world_size))
    return ShardPlan(total_numel, sizes, offsets)


def fsdp2_chunk_plan(params: Sequence, world_size: int) -> ShardPlan:
    """Per-parameter even chunks: rank ``r`` holds
    ``[offset_p + r*n_p/W, +n_p/W)`` of every parameter, stored back to back
    in parameter order (matrix_fsdp/planning/planner.py:428-487).  For a
    row-major ``R x C`` matrix with ``W | R`` this is the row split
    ``rows [r*R/W, (r+1)*R/W)``."""
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, got {world_size}.")
    segments: list[list[LayoutSegment]] = [[] for _ in range(world_size)]
    local = 0
    for p in params:
        if p.numel % world_size:
            raise ValueError(
                f"fsdp2_chunk_plan requires parameter {p.fqn!r} numel={p.numel} "
                f"to be divisible by world_size={world_size}."
            )
        chunk = p.numel // world_size
        for r in range(world_size):
            start = p.offset + r * chunk
            segments[r].append(LayoutSegment(start, start + chunk, local))
        local += chunk
    return ShardPlan.from_rank_segments(sum(p.numel for p in params), segments)


def block_grid_plan(params: Sequence, grid: tuple[int, int]) -> ShardPlan:
    """``gr x gc`` block split of every matrix, rank ``r = i*gc + j`` holding
    block ``(i, j)`` row by row; vectors are cut into ``gr*gc`` contiguous
    parts.  For a matrix ``R x C`` at flat offset ``off`` the rank's segments
    are, for ``rho`` in ``[i*R/gr, (i+1)*R/gr)``::

        global_start = off + rho*C + j*C/gc,  numel = C/gc,
        local_start  = base_p + (rho - i*R/gr) * C/gc

    with ``base_p`` the sum of ``n_q/(gr*gc)`` over the parameters before it.
    The local shard of a matrix is therefore the contiguous copy of
    ``full.view(R, C)[i*R/gr:(i+1)*R/gr, j*C/gc:(j+1)*C/gc]``.  This layout uses
    the reference's segment vocabulary (matrix_fsdp/core/layout.py:15-30) with
    many segments per parameter per rank, which the reference only supports
    through its segment-copy primitives
    (matrix_fsdp/runtime/flat_buffer.py:1304-1333)."""
    gr, gc = grid
    world = gr * gc
    if gr <= 0 or gc <= 0:
        raise ValueError(f"grid must be positive, got {grid}.")
    segments: list[list[LayoutSegment]] = [[] for _ in range(world)]
    base = 0
    for p in params:
        shape = tuple(p.shape)
        if p.numel % world:
            raise ValueError(f"block_grid_plan requires parameter {p.fqn!r} numel={p.numel} divisible by {world}.")
        if len(shape) == 2 and shape[0] % gr == 0 and shape[1] % gc == 0:
            rows, cols = shape
            br, bc = rows // gr, cols // gc
            for r in range(world):
                i, j = divmod(r, gc)
                first = p.offset + i * br * cols + j * bc
                if gc == 1:
                    segments[r].append(LayoutSegment(first, first + br * cols, base))
                    continue
                segments[r].extend(
                    LayoutSegment(first + k * cols, first + k * cols + bc, base + k * bc) for k in range(br)
                )
        else:
            part = p.numel // world
            for r in range(world):
                start = p.offset + r * part
                segments[r].append(LayoutSegment(start, start + part, base))
        base += p.numel // world
    return ShardPlan.from_rank_segments(sum(p.numel for p in params), segments)


def whole_param_owner_plan(params: Sequence, world_size: int, owner_ranks: Sequence[int]) -> ShardPlan:
    """Every parameter lives whole on one owner rank, in parameter order on
    that rank (matrix_fsdp/planning/planner.py:342-387, without merging)."""
    if len(owner_ranks) != len(params):
        raise ValueError("one owner rank per parameter is required.")
    segments: list[list[LayoutSegment]] = [[] for _ in range(world_size)]
    sizes = [0] * world_size
    for p, owner in zip(params, owner_ranks):
        if not 0 <= owner < world_size:
            raise ValueError(f"Owner rank for parameter {p.fqn!r} must be in [0, {world_size}), got {owner}.")
        segments[owner].append(LayoutSegment(p.offset, p.end, sizes[owner]))
        sizes[owner] += p.numel
    return ShardPlan.from_rank_segments(sum(p.numel for p in params), segments)


def rank_major_owner_order(params: Sequence, world_size: int, owner_ranks: Sequence[int]) -> list[int]:
    """Parameter order after the runtime's flat reorder of whole-parameter
    owner layouts: rank 0's parameters first, then rank 1's, ..., each rank's
    in their planner ``local_start`` order (matrix_fsdp/runtime/fsdp_unit.py:1602-1692).
    Re-assigning flat offsets in this order makes every rank's shard one
    contiguous range, so compact rank-major order equals full-buffer order."""
    order: list[int] = []
    for r in range(world_size):
        order.extend(i for i, owner in enumerate(owner_ranks) if owner == r)
    if len(order) != len(params):
        raise ValueError("owner ranks outside [0, world_size).")
    return order


def flat_reordered_owner_layout(params: Sequence, world_size: int, owner_ranks: Sequence[int]):
    """What the runtime executes for a whole-parameter owner layout
    (matrix_fsdp/runtime/fsdp_unit.py:1625-1692): the flat buffer is re-laid
    out rank-major -- rank 0's parameters first, then rank 1's, each rank's in
    their planner order -- so that every rank's shard is ONE contiguous range
    ``(rank_start, rank_end, 0)`` and compact rank-major order equals
    full-buffer order.  Returns ``(order, offsets, plan)``: the parameter
    indices in their new flat order, the new ``(offset, end)`` of every
    parameter (indexed like ``params``) and the shard plan."""
    order = rank_major_owner_order(params, world_size, owner_ranks)
    offsets: list[tuple[int, int]] = [(0, 0)] * len(params)
    segments: list[tuple[LayoutSegment, ...]] = []
    cursor = 0
    for rank in range(world_size):
        start = cursor
        for i in order:
            if owner_ranks[i] == rank:
                offsets[i] = (cursor, cursor + params[i].numel)
                cursor += params[i].numel
        segments.append((LayoutSegment(start, cursor, 0),) if cursor > start else ())
    return order, offsets, ShardPlan.from_rank_segments(cursor, segments)
