"""Group layouts cut at legal boundaries: whole parameters, 1-D blocks, matrix row blocks.

A *block* is a stretch ``[global_start, global_end)`` of one parameter that must
stay on one rank (matrix_fsdp/planning/planner.py:33-43).  A block builder turns
a parameter into its blocks; ``ordered_group_plan`` strings the blocks of an
ordered parameter list together and cuts the string into one run per rank, each
cut at the block boundary nearest to the even split (planner.py:490-533,
913-941).  ``hinted_ordered_group_plan`` picks the builder per parameter from its
``ParamShardHint`` (planner.py:536-574, 651-698) -- the route
``fully_shard(shard_placement_fn=lambda p: Shard(0))`` takes.

The other whole-parameter producers of the reference's planner that the owner
layouts do not cover live here too: ``parameter_boundary_plan`` (planner.py:72-126),
``expert_owner_tail_plan`` (:274-339) and ``rotate_layout_ranks`` (:577-633).

Everything returns a ``MatrixGroupLayout``.
"""
from __future__ import annotations

from dataclasses import dataclass
from itertools import accumulate
from types import SimpleNamespace
from typing import Callable, Sequence

from ..core.layout import LayoutSegment, MatrixGroupLayout, ShardPlan
from ..core.managed_param import ParamRuntimeKind, ParamShardHint
from .owner_plans import _check_world, _fixed_owner, _initial_units, _lightest, whole_param_assignment_plan


@dataclass(frozen=True)
class ParamBlock:
    fqn: str
    global_start: int
    global_end: int
    block_index: int
    kind: str = "block"

    @property
    def numel(self) -> int:
        return self.global_end - self.global_start


BlockBuilder = Callable[[object], Sequence[ParamBlock]]
BlockSizeFn = Callable[[object], int]
RowBlockFn = Callable[[object], int]

_WHOLE = ("parameter", "matrix_owner")
_GRANULARITIES = ("parameter", "matrix_owner", "block", "row_block")


def _hint_of(param) -> ParamShardHint:
    return getattr(param, "shard_hint", None) or ParamShardHint()


def order_params(params: Sequence, order_policy: str = "default") -> list:
    """``default`` keeps the given order, ``largest_first`` sorts by size (ties by
    offset), ``offset`` by flat-buffer position (planner.py:59-69)."""
    if order_policy == "default":
        return list(params)
    if order_policy == "largest_first":
        return sorted(params, key=lambda p: (-p.numel, p.offset))
    if order_policy == "offset":
        return sorted(params, key=lambda p: p.offset)
    raise ValueError(f"Unknown order_policy={order_policy!r}.")


# ---------------------------------------------------------------------------
# Block builders


def whole_param_blocks(param) -> tuple[ParamBlock, ...]:
    return (ParamBlock(param.fqn, param.offset, param.end, 0, "parameter"),)


def _cut_every(param, step: int, kind: str) -> tuple[ParamBlock, ...]:
    """Blocks of ``step`` elements from the parameter's start; the last one ends
    with the parameter."""
    return tuple(
        ParamBlock(param.fqn, start, min(start + step, param.end), index, kind)
        for index, start in enumerate(range(param.offset, param.end, step))
    )


def _hinted_block_units(hint: ParamShardHint) -> int | None:
    if hint.block_shape is None or hint.split_granularity != "block":
        return None
    if len(hint.block_shape) != 1:
        raise ValueError(f"block split_granularity expects a 1D block_shape, got {hint.block_shape}.")
    return hint.block_shape[0]


def _hinted_row_block(hint: ParamShardHint) -> int | None:
    if hint.block_shape is None or hint.split_granularity != "row_block":
        return None
    if len(hint.block_shape) not in (1, 2):
        raise ValueError(f"row_block split_granularity expects a 1D or 2D block_shape, got {hint.block_shape}.")
    return hint.block_shape[0]


def uniform_block_builder(block_size_fn: BlockSizeFn, *, kind: str = "uniform") -> BlockBuilder:
    """Equal blocks; the size comes from a ``block`` hint's ``block_shape`` when
    the parameter has one, else from ``block_size_fn``, and must divide the
    parameter (planner.py:740-765)."""

    def build(param) -> tuple[ParamBlock, ...]:
        hint = _hint_of(param)
        if hint.split_granularity in _WHOLE:
            return whole_param_blocks(param)
        size = _hinted_block_units(hint) or block_size_fn(param)
        if size <= 0:
            raise ValueError(f"block_size_fn returned {size} for {param.fqn}.")
        if param.numel % size:
            raise ValueError(f"Parameter {param.fqn} numel={param.numel} is not divisible by block_size={size}.")
        return _cut_every(param, size, kind)

    return build


def bounded_block_builder(block_size_fn: BlockSizeFn, *, kind: str = "block") -> BlockBuilder:
    """Blocks of at most ``block_size_fn(param)`` elements, a shorter one at the
    end allowed -- unless the parameter carries a ``block`` hint, which stays
    strict (planner.py:713-737)."""
    strict = uniform_block_builder(block_size_fn, kind=kind)

    def build(param) -> tuple[ParamBlock, ...]:
        hint = _hint_of(param)
        if hint.split_granularity in _WHOLE:
            return whole_param_blocks(param)
        if hint.split_granularity == "block":
            return strict(param)
        size = block_size_fn(param)
        if size <= 0:
            raise ValueError(f"block_size_fn returned {size} for {param.fqn}.")
        return _cut_every(param, size, kind)

    return build


def _matrix_dims(param) -> tuple[int, int]:
    if len(param.shape) != 2:
        raise ValueError(f"Parameter {param.fqn} must be 2D for matrix row blocks, got shape={tuple(param.shape)}.")
    rows, cols = tuple(param.shape)
    return int(rows), int(cols)


def matrix_row_block_builder(row_block_fn: RowBlockFn, *, kind: str = "matrix_row_block") -> BlockBuilder:
    """Blocks of whole rows; the row count per block comes from a ``row_block``
    hint when there is one, else from ``row_block_fn``, and must divide the rows
    (planner.py:799-828)."""

    def build(param) -> tuple[ParamBlock, ...]:
        hint = _hint_of(param)
        if hint.split_granularity in _WHOLE:
            return whole_param_blocks(param)
        rows, cols = _matrix_dims(param)
        row_block = _hinted_row_block(hint) or row_block_fn(param)
        if row_block <= 0:
            raise ValueError(f"row_block_fn returned {row_block} for {param.fqn}.")
        if rows % row_block:
            raise ValueError(f"Parameter {param.fqn} rows={rows} is not divisible by row_block={row_block}.")
        return _cut_every(param, row_block * cols, kind)

    return build


def bounded_matrix_row_block_builder(row_block_fn: RowBlockFn, *, kind: str = "matrix_row_block") -> BlockBuilder:
    """Row blocks with a shorter last block allowed, strict again under a
    ``row_block`` hint (planner.py:768-796)."""
    strict = matrix_row_block_builder(row_block_fn, kind=kind)

    def build(param) -> tuple[ParamBlock, ...]:
        hint = _hint_of(param)
        if hint.split_granularity in _WHOLE:
            return whole_param_blocks(param)
        if hint.split_granularity == "row_block":
            return strict(param)
        _, cols = _matrix_dims(param)
        row_block = row_block_fn(param)
        if row_block <= 0:
            raise ValueError(f"row_block_fn returned {row_block} for {param.fqn}.")
        return _cut_every(param, row_block * cols, kind)

    return build


def hint_aware_block_builder(
    *,
    default_granularity: str = "parameter",
    target_block_units: int | None = None,
    row_block_units: int | RowBlockFn | None = None,
    block_kind: str = "block",
) -> BlockBuilder:
    """The parameter's own ``split_granularity`` decides, ``default_granularity``
    where it has none.  A hinted granularity is strict (sizes must divide); a
    defaulted one may leave a shorter last block, and a defaulted ``row_block``
    keeps non-matrices whole (planner.py:651-698).  Without explicit sizes a
    block is the whole parameter and a row block all its rows (:865-876)."""
    if default_granularity not in _GRANULARITIES:
        raise ValueError(f"Unknown default_granularity={default_granularity!r}. Valid granularities: {', '.join(sorted(_GRANULARITIES))}.")
    if target_block_units is not None and target_block_units <= 0:
        raise ValueError(f"target_block_units must be positive, got {target_block_units}.")
    if isinstance(row_block_units, int) and row_block_units <= 0:
        raise ValueError(f"row_block_units must be positive, got {row_block_units}.")

    def block_units(param) -> int:
        return target_block_units or max(1, param.numel)

    def rows_per_block(param) -> int:
        if callable(row_block_units):
            return row_block_units(param)
        if row_block_units is not None:
            return row_block_units
        return max(1, tuple(param.shape)[0]) if len(param.shape) == 2 else 1

    builders = {
        ("block", True): uniform_block_builder(block_units, kind=block_kind),
        ("block", False): bounded_block_builder(block_units, kind=block_kind),
        ("row_block", True): matrix_row_block_builder(rows_per_block),
        ("row_block", False): bounded_matrix_row_block_builder(rows_per_block),
    }

    def build(param) -> tuple[ParamBlock, ...]:
        hinted = _hint_of(param).split_granularity
        granularity = hinted or default_granularity
        if granularity in _WHOLE:
            return whole_param_blocks(param)
        if granularity not in ("block", "row_block"):
            raise ValueError(f"Unknown split_granularity={granularity!r} for parameter {param.fqn}.")
        if granularity == "row_block" and hinted is None and len(param.shape) != 2:
            return whole_param_blocks(param)
        return builders[(granularity, hinted is not None)](param)

    return build


def validate_param_blocks(param, blocks: Sequence[ParamBlock]) -> None:
    """Blocks must tile ``[param.offset, param.end)`` exactly, each with its own
    index (planner.py:891-910)."""
    cursor = param.offset
    indices: set[int] = set()
    for block in sorted(blocks, key=lambda b: (b.global_start, b.global_end)):
        if block.fqn != param.fqn:
            raise ValueError(f"Block for {block.fqn} cannot be used for parameter {param.fqn}.")
        if block.block_index in indices:
            raise ValueError(f"Parameter {param.fqn} has duplicate block_index={block.block_index}.")
        indices.add(block.block_index)
        if block.global_start < param.offset or block.global_end > param.end:
            raise ValueError(f"Block {block} crosses parameter {param.fqn} boundary.")
        if block.global_start < cursor:
            raise ValueError(f"Parameter {param.fqn} blocks overlap at {block}.")
        if block.global_start > cursor:
            raise ValueError(f"Parameter {param.fqn} blocks have gap before {block}.")
        if block.numel <= 0:
            raise ValueError(f"Parameter {param.fqn} has empty block {block}.")
        cursor = block.global_end
    if cursor != param.end:
        raise ValueError(f"Parameter {param.fqn} block coverage ends at {cursor}, expected {param.end}.")


# ---------------------------------------------------------------------------
# Cutting an ordered run of blocks into one stretch per rank


def split_points(block_sizes: Sequence[int], world_size: int) -> list[int]:
    """``cuts[r]`` = number of leading blocks that ranks ``0..r`` hold together.

    Rank ``r`` (not the last) aims at ``round(total * (r + 1) / world_size)``
    elements behind it -- Python's round, halves to even -- and takes blocks
    while that brings the running total no further from the aim, stopping once
    the aim is reached; it always takes one block if any is left.  The last rank
    takes the rest (planner.py:913-941)."""
    ends = list(accumulate(block_sizes))
    total = ends[-1] if ends else 0
    cuts: list[int] = []
    taken = 0
    for rank in range(world_size - 1):
        aim = round(total * (rank + 1) / world_size)
        first = taken
        while taken < len(ends):
            have = ends[taken - 1] if taken else 0
            if taken > first and abs(ends[taken] - aim) > abs(have - aim):
                break
            taken += 1
            if ends[taken - 1] >= aim:
                break
        cuts.append(taken)
    cuts.append(len(ends))
    return cuts


def _segments_of(blocks: Sequence[ParamBlock]) -> tuple[LayoutSegment, ...]:
    """Blocks that continue each other in the flat buffer merge into one segment."""
    spans: list[list[int]] = []
    for block in blocks:
        if spans and spans[-1][1] == block.global_start:
            spans[-1][1] = block.global_end
        else:
            spans.append([block.global_start, block.global_end])
    local_starts = accumulate((end - start for start, end in spans), initial=0)
    return tuple(LayoutSegment(start, end, local) for (start, end), local in zip(spans, local_starts))


def ordered_group_plan(
    params: Sequence,
    world_size: int,
    *,
    block_builder: BlockBuilder | None = None,
    block_size_fn: BlockSizeFn | None = None,
    order_policy: str = "default",
) -> MatrixGroupLayout:
    """Rank-contiguous cut of the ordered parameters at block boundaries; one block
    per parameter unless a builder or a block size is given (planner.py:490-533)."""
    _check_world(world_size)
    if block_builder is not None and block_size_fn is not None:
        raise ValueError("Pass only one of block_builder or block_size_fn.")
    ordered = order_params(params, order_policy)
    total = sum(p.numel for p in params)
    if total == 0:
        return MatrixGroupLayout.from_rank_segments(0, tuple(() for _ in range(world_size)))
    if block_builder is None:
        block_builder = whole_param_blocks if block_size_fn is None else uniform_block_builder(block_size_fn)
    blocks: list[ParamBlock] = []
    for param in ordered:
        mine = tuple(block_builder(param))
        validate_param_blocks(param, mine)
        blocks.extend(mine)
    cuts = split_points([b.numel for b in blocks], world_size)
    rank_segments = tuple(_segments_of(blocks[lo:hi]) for lo, hi in zip([0] + cuts[:-1], cuts))
    return MatrixGroupLayout.from_shard_plan(ShardPlan.from_rank_segments(total, rank_segments), params)


def hinted_ordered_group_plan(
    params: Sequence,
    world_size: int,
    *,
    default_granularity: str = "parameter",
    target_block_units: int | None = None,
    row_block_units: int | RowBlockFn | None = None,
    block_kind: str = "block",
    order_policy: str = "default",
) -> MatrixGroupLayout:
    """``ordered_group_plan`` with the blocks each parameter's ``ParamShardHint``
    asks for (planner.py:536-574)."""
    builder = hint_aware_block_builder(
        default_granularity=default_granularity,
        target_block_units=target_block_units,
        row_block_units=row_block_units,
        block_kind=block_kind,
    )
    return ordered_group_plan(params, world_size, block_builder=builder, order_policy=order_policy)


# ---------------------------------------------------------------------------
# Whole-parameter producers


def parameter_boundary_plan(params: Sequence, world_size: int, *, order_policy: str = "default") -> MatrixGroupLayout:
    """Every parameter whole, each to the rank that is lightest when its turn
    comes (planner.py:72-126)."""
    _check_world(world_size)
    units = [0] * world_size
    assignments = []
    for param in order_params(params, order_policy):
        rank = _lightest(units)
        assignments.append((param, rank))
        units[rank] += param.numel
    return MatrixGroupLayout.from_shard_plan(whole_param_assignment_plan(params, world_size, assignments), params)


def expert_owner_tail_plan(
    params: Sequence,
    world_size: int,
    *,
    initial_rank_units: Sequence[int] | None = None,
    dense_order_policy: str = "largest_first",
    merge_adjacent_rank_segments: bool = True,
) -> MatrixGroupLayout:
    """All parameters of one routed expert (``runtime_kind="expert_owner"`` or an
    ``expert_group_id``) stay on one rank: expert groups go first, largest first,
    each to the lightest rank (or the rank an ``owner_rank`` hint fixes), then the
    remaining parameters fill up the lightest ranks one by one (planner.py:274-339)."""
    _check_world(world_size)
    units = _initial_units(initial_rank_units, world_size)
    experts: dict[str, list] = {}
    others: list = []
    for param in params:
        hint = _hint_of(param)
        if hint.runtime_kind == ParamRuntimeKind.EXPERT_OWNER or hint.expert_group_id:
            experts.setdefault(hint.expert_group_id or param.fqn, []).append(param)
        else:
            others.append(param)
    roles = sorted(experts.values(), key=lambda group: (-sum(p.numel for p in group), min(p.offset for p in group)))
    roles += [[param] for param in order_params(others, dense_order_policy)]
    assignments = []
    for role in roles:
        fixed = _fixed_owner(role, world_size)
        rank = _lightest(units) if fixed is None else fixed
        assignments.extend((param, rank) for param in role)
        units[rank] += sum(p.numel for p in role)
    plan = whole_param_assignment_plan(params, world_size, assignments, merge_adjacent_rank_segments=merge_adjacent_rank_segments)
    return MatrixGroupLayout.from_shard_plan(plan, params)


def rotate_layout_ranks(layout: MatrixGroupLayout, rank_offset: int) -> MatrixGroupLayout:
    """Rank ``r``'s shard moves to rank ``(r + rank_offset) % world_size`` as it
    is, so that a row of alike units does not pile its matrices on the same
    ranks (planner.py:577-633)."""
    world = layout.world_size
    if world <= 0 or rank_offset % world == 0:
        return layout
    shift = rank_offset % world
    rolled = tuple(layout.rank_segments[(rank - shift) % world] for rank in range(world))
    spans = [SimpleNamespace(fqn=p.fqn, offset=p.global_start, end=p.global_end) for p in layout.params]
    return MatrixGroupLayout.from_shard_plan(ShardPlan.from_rank_segments(layout.total_numel, rolled), spans)
