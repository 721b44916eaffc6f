"""Block / row-block group planners, the layout validator and shard-hint validation against the literal
expectations of the reference's own tests (test/fsdp/test_planner.py, test_layout_validator.py,
test_managed_param.py), plus brute-force properties of the rank cut on random inputs."""
import random
from dataclasses import dataclass

import pytest
import torch
from torch import nn

from matrix_fsdp_amd.core.layout import LayoutSegment, MatrixGroupLayout, ParamLayout, ParamSegment, RankLayout
from matrix_fsdp_amd.core.managed_param import ManagedParamRegistry, ParamRuntimeKind, ParamShardHint
from matrix_fsdp_amd.core.placement import matrix_shard_from_layout
from matrix_fsdp_amd.core.plans import contiguous_even_plan, fsdp2_chunk_plan
from matrix_fsdp_amd.planning import (
    ParamBlock,
    bounded_block_builder,
    bounded_matrix_row_block_builder,
    expert_owner_tail_plan,
    explain_runtime_layout_compatibility,
    hinted_ordered_group_plan,
    matrix_row_block_builder,
    ordered_group_plan,
    parameter_boundary_plan,
    rotate_layout_ranks,
    split_points,
    uniform_block_builder,
    validate_group_layout,
    validate_runtime_layout,
    whole_param_blocks,
)


@dataclass(frozen=True)
class P:
    fqn: str
    numel: int
    offset: int
    shape: tuple = None
    shard_hint: ParamShardHint = ParamShardHint()

    def __post_init__(self):
        if self.shape is None:
            object.__setattr__(self, "shape", (self.numel,))

    @property
    def end(self):
        return self.offset + self.numel


S = LayoutSegment


# ---------------------------------------------------------------- test_planner.py:43-125
def test_contiguous_even_plan():
    plan = contiguous_even_plan(10, 4)
    assert plan.shard_sizes == (3, 3, 2, 2) and plan.shard_offsets == (0, 3, 6, 8)
    assert plan.local_range(2) == (6, 8) and plan.local_segments(2) == (S(6, 8, 0),)
    with pytest.raises(ValueError, match="world_size must be positive"):
        contiguous_even_plan(10, 0)


def test_parameter_boundary_plan():
    params = (P("p0", 5, 0), P("p1", 4, 5), P("p2", 3, 9), P("p3", 2, 12))
    layout = parameter_boundary_plan(params, 2)
    assert layout.total_numel == 14 and layout.shard_sizes == (7, 7)
    assert layout.rank_segments == ((S(0, 5, 0), S(12, 14, 5)), (S(5, 9, 0), S(9, 12, 4)))
    assert tuple(p.fqn for p in layout.params) == ("p0", "p1", "p2", "p3")
    assert layout.owner_ranks("p0") == (0,) and layout.owner_ranks("p1") == (1,)
    assert layout.params_for_rank(0) == ("p0", "p3")
    assert layout.rank_segments_for_param(0, "p3") == (ParamSegment("p3", 0, 12, 14, 5),)
    assert layout.to_shard_plan().local_segments(0) == layout.rank_segments[0]

    params = (P("small0", 1, 0), P("large", 8, 1), P("small1", 1, 9))
    default, largest = parameter_boundary_plan(params, 2), parameter_boundary_plan(params, 2, order_policy="largest_first")
    assert default.params_for_rank(0) == ("small0", "small1") and default.params_for_rank(1) == ("large",)
    assert largest.params_for_rank(0) == ("large",) and largest.params_for_rank(1) == ("small0", "small1")
    with pytest.raises(ValueError, match="Unknown order_policy"):
        parameter_boundary_plan((), 1, order_policy="unknown")
    with pytest.raises(ValueError, match="world_size must be positive"):
        parameter_boundary_plan((), 0)


def test_rotate_layout_ranks():
    params = (P("p0", 5, 0), P("p1", 4, 5), P("p2", 3, 9))
    layout = parameter_boundary_plan(params, 3)
    rotated = rotate_layout_ranks(layout, 1)
    assert rotated.total_numel == layout.total_numel and rotated.shard_sizes == (3, 5, 4)
    assert [rotated.owner_ranks(n) for n in ("p0", "p1", "p2")] == [(1,), (2,), (0,)]
    assert rotated.rank_segments == ((S(9, 12, 0),), (S(0, 5, 0),), (S(5, 9, 0),))
    validate_group_layout(rotated, params, 3)
    assert rotate_layout_ranks(layout, 3) is layout
    assert rotate_layout_ranks(rotated, -1).rank_segments == layout.rank_segments
    # several segments per rank keep their order and local offsets
    two = parameter_boundary_plan((P("a", 5, 0), P("b", 4, 5), P("c", 3, 9), P("d", 2, 12)), 2)
    swapped = rotate_layout_ranks(two, 1)
    assert swapped.rank_segments == (two.rank_segments[1], two.rank_segments[0])
    assert swapped.rank_segments_for_param(1, "d") == (ParamSegment("d", 1, 12, 14, 5),)


# ---------------------------------------------------------------- test_planner.py:127-226
def test_expert_owner_tail_plan():
    def expert(name, offset, shape, eid):
        hint = ParamShardHint(
            optimizer_type="muon", split_granularity="matrix_owner", runtime_kind=ParamRuntimeKind.EXPERT_OWNER, expert_id=eid, expert_group_id=f"moe.experts.{eid}"
        )
        return P(name, 8, offset, shape, hint)

    params = (
        P("dense.weight", 10, 0, (2, 5)),
        expert("moe.experts.0.w1.weight", 10, (2, 4), 0),
        expert("moe.experts.0.w2.weight", 18, (4, 2), 0),
        expert("moe.experts.1.w1.weight", 26, (2, 4), 1),
        expert("moe.experts.1.w2.weight", 34, (4, 2), 1),
        P("moe.router.weight", 2, 42, (1, 2), ParamShardHint(optimizer_type="adamw", split_granularity="parameter")),
    )
    layout = expert_owner_tail_plan(params, 2)
    assert layout.owner_ranks("moe.experts.0.w1.weight") == layout.owner_ranks("moe.experts.0.w2.weight") == (0,)
    assert layout.owner_ranks("moe.experts.1.w1.weight") == layout.owner_ranks("moe.experts.1.w2.weight") == (1,)
    assert layout.owner_ranks("dense.weight") == (0,) and layout.owner_ranks("moe.router.weight") == (1,)
    assert layout.shard_sizes == (26, 18)
    validate_group_layout(layout, params, 2)
    # rank 1 starts heavier: the first expert still goes to rank 0, the second one too
    skewed = expert_owner_tail_plan(params, 2, initial_rank_units=(0, 100))
    assert skewed.shard_sizes == (44, 0)
    with pytest.raises(ValueError, match="initial_rank_units length"):
        expert_owner_tail_plan(params, 2, initial_rank_units=(0,))


def test_fsdp2_chunk_plan():
    plan = fsdp2_chunk_plan((P("p0", 6, 0), P("p1", 4, 6)), 2)
    assert plan.total_numel == 10 and plan.shard_sizes == (5, 5)
    assert plan.rank_segments == ((S(0, 3, 0), S(6, 8, 3)), (S(3, 6, 0), S(8, 10, 3)))
    with pytest.raises(ValueError, match="divisible"):
        fsdp2_chunk_plan((P("p0", 5, 0),), 2)


# ---------------------------------------------------------------- test_planner.py:228-294, 421-493
def test_ordered_group_plan():
    params = (P("p0", 5, 0), P("p1", 4, 5), P("p2", 3, 9), P("p3", 2, 12))
    layout = ordered_group_plan(params, 2)
    assert layout.shard_sizes == (9, 5) and layout.rank_segments == ((S(0, 9, 0),), (S(9, 14, 0),))
    assert layout.params_for_rank(0) == ("p0", "p1") and layout.params_for_rank(1) == ("p2", "p3")
    validate_group_layout(layout, params, 2)

    params = (P("p0", 6, 0), P("p1", 6, 6))
    layout = ordered_group_plan(params, 3, block_size_fn=lambda p: 3)
    assert layout.shard_sizes == (3, 6, 3)
    assert layout.rank_segments == ((S(0, 3, 0),), (S(3, 9, 0),), (S(9, 12, 0),))
    assert layout.owner_ranks("p0") == (0, 1) and layout.owner_ranks("p1") == (1, 2)
    assert layout.rank_segments_for_param(1, "p0") == (ParamSegment("p0", 1, 3, 6, 0),)
    assert layout.rank_segments_for_param(1, "p1") == (ParamSegment("p1", 1, 6, 9, 3),)
    validate_group_layout(layout, params, 3)

    params = (P("p0", 8, 0), P("p1", 4, 8))
    four = lambda p: tuple(ParamBlock(p.fqn, s, s + 4, i, "matrix_row_block") for i, s in enumerate(range(p.offset, p.end, 4)))  # noqa: E731
    layout = ordered_group_plan(params, 2, block_builder=four)
    assert layout.shard_sizes == (8, 4) and layout.rank_segments == ((S(0, 8, 0),), (S(8, 12, 0),))
    assert layout.owner_ranks("p0") == (0,) and layout.owner_ranks("p1") == (1,)

    params = (P("w0", 24, 0, (6, 4)), P("w1", 8, 24, (2, 4)))
    layout = ordered_group_plan(params, 2, block_builder=matrix_row_block_builder(lambda p: 2))
    assert layout.shard_sizes == (16, 16) and layout.rank_segments == ((S(0, 16, 0),), (S(16, 32, 0),))
    assert layout.owner_ranks("w0") == (0, 1) and layout.owner_ranks("w1") == (1,)
    validate_group_layout(layout, params, 2)

    empty = ordered_group_plan((), 3)
    assert empty.total_numel == 0 and empty.shard_sizes == (0, 0, 0)


def test_ordered_group_plan_rejections():
    one = (P("p0", 4, 0),)
    with pytest.raises(ValueError, match="Pass only one"):
        ordered_group_plan(one, 2, block_builder=lambda p: (ParamBlock(p.fqn, p.offset, p.end, 0),), block_size_fn=lambda p: p.numel)
    with pytest.raises(ValueError, match="not divisible"):
        ordered_group_plan((P("p0", 5, 0),), 2, block_size_fn=lambda p: 2)
    with pytest.raises(ValueError, match="block_size_fn returned"):
        ordered_group_plan((P("p0", 5, 0),), 2, block_size_fn=lambda p: 0)
    with pytest.raises(ValueError, match="world_size must be positive"):
        ordered_group_plan((), 0)
    eight = (P("p0", 8, 0),)
    for blocks, message in [
        (((0, 4, 0), (5, 8, 1)), "gap"),
        (((0, 5, 0), (4, 8, 1)), "overlap"),
        (((0, 9, 0),), "crosses"),
        (((0, 4, 0), (4, 8, 0)), "duplicate"),
        (((0, 4, 0),), "coverage ends at 4"),
    ]:
        with pytest.raises(ValueError, match=message):
            ordered_group_plan(eight, 2, block_builder=lambda p, blocks=blocks: tuple(ParamBlock(p.fqn, a, b, i) for a, b, i in blocks))


# ---------------------------------------------------------------- test_planner.py:296-419
def test_block_builders():
    p = P("p0", 8, 3)
    assert whole_param_blocks(p) == (ParamBlock("p0", 3, 11, 0, "parameter"),)
    assert uniform_block_builder(lambda c: 2, kind="quant_block")(p) == tuple(ParamBlock("p0", 3 + 2 * i, 5 + 2 * i, i, "quant_block") for i in range(4))
    hinted = P("p0", 8, 3, shard_hint=ParamShardHint(split_granularity="block", block_shape=(4,)))
    assert uniform_block_builder(lambda c: 2, kind="quant_block")(hinted) == (ParamBlock("p0", 3, 7, 0, "quant_block"), ParamBlock("p0", 7, 11, 1, "quant_block"))
    ten = P("p0", 10, 3)
    assert bounded_block_builder(lambda c: 4, kind="ordered_block")(ten) == (
        ParamBlock("p0", 3, 7, 0, "ordered_block"),
        ParamBlock("p0", 7, 11, 1, "ordered_block"),
        ParamBlock("p0", 11, 13, 2, "ordered_block"),
    )
    with pytest.raises(ValueError, match="not divisible"):
        bounded_block_builder(lambda c: 4)(P("p0", 10, 3, shard_hint=ParamShardHint(split_granularity="block", block_shape=(4,))))


def test_matrix_row_block_builders():
    w = P("w", 24, 10, (6, 4))
    rows2 = matrix_row_block_builder(lambda c: 2)
    assert rows2(w) == tuple(ParamBlock("w", 10 + 8 * i, 18 + 8 * i, i, "matrix_row_block") for i in range(3))
    owner = P("w", 24, 10, (6, 4), ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner"))
    assert rows2(owner) == whole_param_blocks(owner)
    hinted = P("w", 24, 10, (6, 4), ParamShardHint(split_granularity="row_block", block_shape=(3, 4)))
    assert rows2(hinted) == (ParamBlock("w", 10, 22, 0, "matrix_row_block"), ParamBlock("w", 22, 34, 1, "matrix_row_block"))
    with pytest.raises(ValueError, match="must be 2D"):
        rows2(P("bias", 8, 0, (8,)))
    with pytest.raises(ValueError, match="not divisible"):
        matrix_row_block_builder(lambda c: 4)(P("w", 24, 0, (6, 4)))
    with pytest.raises(ValueError, match="row_block_fn returned"):
        matrix_row_block_builder(lambda c: 0)(P("w", 24, 0, (6, 4)))
    five = P("w", 20, 10, (5, 4))
    assert bounded_matrix_row_block_builder(lambda c: 2)(five) == (
        ParamBlock("w", 10, 18, 0, "matrix_row_block"),
        ParamBlock("w", 18, 26, 1, "matrix_row_block"),
        ParamBlock("w", 26, 30, 2, "matrix_row_block"),
    )


# ---------------------------------------------------------------- test_planner.py:495-561
def test_hinted_ordered_group_plan():
    params = (
        P("muon", 24, 0, (6, 4), ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")),
        P("rows", 24, 24, (6, 4), ParamShardHint(split_granularity="row_block", block_shape=(2, 4))),
        P("blocks", 8, 48, shard_hint=ParamShardHint(split_granularity="block", block_shape=(4,))),
        P("bias", 3, 56),
    )
    layout = hinted_ordered_group_plan(params, 3, default_granularity="parameter")
    assert layout.shard_sizes == (24, 16, 19)
    assert layout.rank_segments == ((S(0, 24, 0),), (S(24, 40, 0),), (S(40, 59, 0),))
    assert [layout.owner_ranks(n) for n in ("muon", "rows", "blocks", "bias")] == [(0,), (1, 2), (2,), (2,)]
    assert matrix_shard_from_layout(layout).local_units == (24, 16, 19)
    validate_group_layout(layout, params, 3)
    assert explain_runtime_layout_compatibility(layout, params, 3).mode == "matrix_shard"

    params = (P("w", 20, 0, (5, 4)), P("bias", 5, 20, (5,)))
    layout = hinted_ordered_group_plan(params, 2, default_granularity="row_block", row_block_units=2)
    assert layout.shard_sizes == (16, 9)
    assert layout.owner_ranks("w") == (0, 1) and layout.owner_ranks("bias") == (1,)
    assert matrix_shard_from_layout(layout).local_units == (16, 9)
    validate_group_layout(layout, params, 2)

    with pytest.raises(ValueError, match="Unknown default_granularity"):
        hinted_ordered_group_plan((P("p0", 4, 0),), 2, default_granularity="unknown")
    with pytest.raises(ValueError, match="target_block_units must be positive"):
        hinted_ordered_group_plan((P("p0", 4, 0),), 2, target_block_units=0)
    # a defaulted block granularity leaves a shorter last block; a callable picks the rows per block
    layout = hinted_ordered_group_plan((P("v", 10, 0),), 2, default_granularity="block", target_block_units=4)
    assert layout.shard_sizes == (4, 6)
    layout = hinted_ordered_group_plan((P("w", 24, 0, (6, 4)),), 3, default_granularity="row_block", row_block_units=lambda p: 1)
    assert layout.shard_sizes == (8, 8, 8)


def test_shard0_hints_cut_between_rows():
    """What ``fully_shard(shard_placement_fn=lambda p: Shard(0))`` plans for ``Sequential(Linear(4, 2), LayerNorm(2))``
    (hints as test_matrix_fsdp_e2e.py:252-268 expects them): 14 elements; two ranks aim at 7 and cut after the
    weight's second row (8); three ranks aim at 5 and 9: one row (4), then the other row and one bias element (5)."""
    module = nn.Sequential(nn.Linear(4, 2), nn.LayerNorm(2))
    hints = {
        "0.weight": ParamShardHint(split_granularity="row_block", block_shape=(1, 4)),
        "0.bias": ParamShardHint(split_granularity="block", block_shape=(1,)),
        "1.weight": ParamShardHint(split_granularity="block", block_shape=(1,)),
        "1.bias": ParamShardHint(split_granularity="block", block_shape=(1,)),
    }
    registry = ManagedParamRegistry.from_module(module, shard_hints=hints)
    layout = hinted_ordered_group_plan(registry.as_list(), 2, default_granularity="parameter")
    assert layout.shard_sizes == (8, 6)
    layout = hinted_ordered_group_plan(registry.as_list(), 3, default_granularity="parameter")
    assert layout.shard_sizes == (4, 5, 5)
    assert explain_runtime_layout_compatibility(layout, registry.as_list(), 3).mode == "matrix_shard"


# ---------------------------------------------------------------- the rank cut itself
def _cut_reference(sizes, world):
    """The rule spelled out on running totals, rank by rank."""
    total, out, i, have = sum(sizes), [], 0, 0
    for rank in range(world - 1):
        aim, first = round(total * (rank + 1) / world), i
        while i < len(sizes) and not (i > first and abs(have + sizes[i] - aim) > abs(have - aim)):
            have += sizes[i]
            i += 1
            if have >= aim:
                break
        out.append(i)
    return out + [len(sizes)]


def test_split_points_properties():
    assert split_points([5, 4, 3, 2], 2) == [2, 4]  # 9 | 5: nine is as near to seven as five, and ties take the block
    assert split_points([3, 3, 3, 3], 3) == [1, 3, 4]
    assert split_points([4], 3) == [1, 1, 1]
    assert split_points([], 2) == [0, 0]
    assert split_points([1, 1, 1], 2) == [2, 3]  # the aim round(1.5) = 2: halves go to even
    assert split_points([1] * 5, 2) == [2, 5]  # round(2.5) = 2
    rng = random.Random(0)
    for _ in range(300):
        sizes = [rng.randint(1, 9) for _ in range(rng.randint(0, 12))]
        world = rng.randint(1, 6)
        cuts = split_points(sizes, world)
        assert cuts == _cut_reference(sizes, world)
        assert len(cuts) == world and cuts[-1] == len(sizes) and all(a <= b for a, b in zip(cuts, cuts[1:]))
        # while blocks are left every rank but the last takes at least one
        for before, after in zip([0] + cuts[:-2], cuts[:-1]):
            assert after > before or before == len(sizes)
    # equal blocks that divide evenly give the even split
    assert split_points([2] * 12, 4) == [3, 6, 9, 12]


def test_random_hinted_plans_are_valid_layouts():
    rng = random.Random(1)
    for _ in range(100):
        params, offset = [], 0
        for i in range(rng.randint(1, 6)):
            kind = rng.choice(["matrix", "vector", "owner"])
            if kind == "vector":
                n = rng.randint(1, 12)
                unit = rng.choice([d for d in range(1, n + 1) if n % d == 0])
                hint = rng.choice([ParamShardHint(), ParamShardHint(split_granularity="block", block_shape=(unit,))])
                params.append(P(f"p{i}", n, offset, (n,), hint))
            else:
                rows, cols = rng.randint(1, 6), rng.randint(1, 5)
                row_block = rng.choice([d for d in range(1, rows + 1) if rows % d == 0])
                hint = ParamShardHint(split_granularity="matrix_owner") if kind == "owner" else ParamShardHint(split_granularity="row_block", block_shape=(row_block, cols))
                params.append(P(f"p{i}", rows * cols, offset, (rows, cols), hint))
            offset = params[-1].end
        world = rng.randint(1, 5)
        layout = hinted_ordered_group_plan(params, world, default_granularity=rng.choice(["parameter", "block", "row_block"]))
        validate_group_layout(layout, params, world)  # includes the hint rules: owners whole, cuts aligned
        assert sum(layout.shard_sizes) == offset
        assert explain_runtime_layout_compatibility(layout, params, world).mode == "matrix_shard"


# ---------------------------------------------------------------- test_layout_validator.py
def _linear_params():
    return ManagedParamRegistry.from_module(nn.Sequential(nn.Linear(4, 2), nn.Linear(2, 1))).as_list()


def _owner_layout(rank1=((8, 10, 0), (10, 13, 2))):
    pieces = (("0.weight", 0, 0, 8, 0), ("0.bias", 1, 8, 10, 0), ("1.weight", 1, 10, 12, 2), ("1.bias", 1, 12, 13, 4))
    return MatrixGroupLayout.from_rank_segments(
        13,
        ((S(0, 8, 0),), tuple(S(*s) for s in rank1)),
        tuple(ParamLayout(n, a, b, (ParamSegment(n, r, a, b, l),)) for n, r, a, b, l in pieces),
    )


def test_runtime_layout_modes():
    params = _linear_params()
    valid = _owner_layout()
    validate_group_layout(valid, params, 2)
    contiguous = explain_runtime_layout_compatibility(_owner_layout(rank1=((8, 13, 0),)), params, 2)
    assert contiguous.compatible and contiguous.mode == "matrix_shard" and not contiguous.requires_flat_reorder
    reorder = explain_runtime_layout_compatibility(valid, params, 2)
    assert reorder.compatible and reorder.mode == "flat_reorder" and reorder.requires_flat_reorder
    refused = explain_runtime_layout_compatibility(valid, params, 2, allow_flat_reorder=False)
    assert not refused.compatible and refused.mode == "unsupported" and refused.requires_flat_reorder
    with pytest.raises(ValueError, match="cannot execute planner layout"):
        validate_runtime_layout(valid, params, 2, allow_flat_reorder=False)

    module = nn.Module()
    module.register_parameter("a", nn.Parameter(torch.empty(8)))
    module.register_parameter("b", nn.Parameter(torch.empty(8)))
    vectors = ManagedParamRegistry.from_module(module).as_list()
    halves = ((S(0, 4, 0), S(8, 12, 4)), (S(4, 8, 0), S(12, 16, 4)))
    split = MatrixGroupLayout.from_rank_segments(
        16,
        halves,
        (
            ParamLayout("a", 0, 8, (ParamSegment("a", 0, 0, 4, 0), ParamSegment("a", 1, 4, 8, 0))),
            ParamLayout("b", 8, 16, (ParamSegment("b", 0, 8, 12, 4), ParamSegment("b", 1, 12, 16, 4))),
        ),
    )
    verdict = explain_runtime_layout_compatibility(split, vectors, 2)
    assert verdict.compatible and verdict.mode == "segment_runtime" and not verdict.requires_flat_reorder
    disabled = explain_runtime_layout_compatibility(split, vectors, 2, allow_segment_runtime=False)
    assert not disabled.compatible and disabled.mode == "unsupported" and "segment_runtime" in disabled.reason

    weight = ManagedParamRegistry.from_module(nn.Linear(16, 1, bias=False)).as_list()
    repeated = MatrixGroupLayout.from_rank_segments(
        16,
        halves,
        (ParamLayout("weight", 0, 16, (ParamSegment("weight", 0, 0, 4, 0), ParamSegment("weight", 1, 4, 8, 0), ParamSegment("weight", 0, 8, 12, 4), ParamSegment("weight", 1, 12, 16, 4))),),
    )
    verdict = explain_runtime_layout_compatibility(repeated, weight, 2)
    assert not verdict.compatible and verdict.mode == "unsupported" and "multiple local segments" in verdict.reason
    with pytest.raises(ValueError, match="cannot execute planner layout"):
        validate_runtime_layout(repeated, weight, 2)


def test_validator_rejections():
    params = _linear_params()
    valid = _owner_layout()

    def with_param(index, layout_param):
        changed = list(valid.params)
        changed[index] = layout_param
        return MatrixGroupLayout(valid.total_numel, valid.ranks, tuple(changed))

    cases = [
        (MatrixGroupLayout(12, valid.ranks, valid.params), "total_numel"),
        (MatrixGroupLayout.from_rank_segments(13, ((S(0, 8, 0),), (S(9, 13, 0),)), valid.params), "rank segments gap"),
        (MatrixGroupLayout(13, valid.ranks, (valid.params[1], valid.params[0], *valid.params[2:])), "do not match managed params"),
        (with_param(0, ParamLayout("0.weight", 0, 8, (ParamSegment("0.weight", 0, 0, 7, 0),))), "param 0.weight coverage"),
        (with_param(0, ParamLayout("0.weight", 0, 8, (ParamSegment("0.weight", 0, 0, 5, 0), ParamSegment("0.weight", 0, 4, 8, 4)))), "param 0.weight overlap"),
        (with_param(0, ParamLayout("0.weight", 0, 8, (ParamSegment("0.weight", 2, 0, 8, 0),))), "invalid rank"),
        (with_param(1, ParamLayout("0.bias", 8, 10, (ParamSegment("0.bias", 1, 7, 10, 0),))), "crosses parameter boundary"),
        (with_param(1, ParamLayout("0.bias", 8, 10, (ParamSegment("0.bias", 1, 8, 10, 1),))), "does not project onto rank"),
        (MatrixGroupLayout(13, (valid.ranks[0], RankLayout(1, 5, (S(8, 10, 1), S(10, 13, 3)))), valid.params), "expected contiguous local_start=0"),
        (MatrixGroupLayout(13, (valid.ranks[0], RankLayout(1, 6, valid.ranks[1].segments)), valid.params), "local_units=6, expected 5"),
        (MatrixGroupLayout(13, valid.ranks[:1], valid.params), "has 1 ranks, expected world_size=2"),
    ]
    for layout, message in cases:
        with pytest.raises(ValueError, match=message):
            validate_group_layout(layout, params, 2)

    def two_halves(name, total=16):
        return MatrixGroupLayout.from_rank_segments(
            total, ((S(0, 8, 0),), (S(8, 16, 0),)), (ParamLayout(name, 0, 16, (ParamSegment(name, 0, 0, 8, 0), ParamSegment(name, 1, 8, 16, 0))),)
        )

    owner = ManagedParamRegistry.from_module(nn.Linear(4, 4, bias=False), shard_hints={"weight": ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")})
    with pytest.raises(ValueError, match="matrix_owner"):
        validate_group_layout(two_halves("weight"), owner.as_list(), 2)
    rows = ManagedParamRegistry.from_module(nn.Linear(4, 4, bias=False), shard_hints={"weight": ParamShardHint(split_granularity="row_block", block_shape=(2, 4))})
    validate_group_layout(two_halves("weight"), rows.as_list(), 2)
    misaligned = MatrixGroupLayout.from_rank_segments(
        16, ((S(0, 4, 0),), (S(4, 16, 0),)), (ParamLayout("weight", 0, 16, (ParamSegment("weight", 0, 0, 4, 0), ParamSegment("weight", 1, 4, 16, 0))),)
    )
    with pytest.raises(ValueError, match="not aligned"):
        validate_group_layout(misaligned, rows.as_list(), 2)
    expert = ParamShardHint(split_granularity="matrix_owner", runtime_kind=ParamRuntimeKind.EXPERT_OWNER, expert_group_id="experts.0")
    pair = ManagedParamRegistry.from_module(nn.Sequential(nn.Linear(4, 2, bias=False), nn.Linear(2, 4, bias=False)), shard_hints={"0.weight": expert, "1.weight": expert})
    spread = MatrixGroupLayout.from_rank_segments(
        16,
        ((S(0, 8, 0),), (S(8, 16, 0),)),
        (ParamLayout("0.weight", 0, 8, (ParamSegment("0.weight", 0, 0, 8, 0),)), ParamLayout("1.weight", 8, 16, (ParamSegment("1.weight", 1, 8, 16, 0),))),
    )
    with pytest.raises(ValueError, match="Expert group"):
        validate_group_layout(spread, pair.as_list(), 2)


# ---------------------------------------------------------------- test_managed_param.py
def test_managed_param_registry_and_hint_validation():
    module = nn.Sequential(nn.Linear(4, 3), nn.Linear(3, 2, bias=False))
    registry = ManagedParamRegistry.from_module(module)
    assert registry.fqns == ("0.weight", "0.bias", "1.weight") and registry.total_numel == 21 and len(registry) == 3
    assert [p.offset for p in registry] == [0, 12, 15] and [p.end for p in registry] == [12, 15, 21]
    assert registry.param("0.weight").param is module[0].weight and registry[2].fqn == "1.weight"
    assert registry.param("0.weight").shard_hint == ParamShardHint()
    with pytest.raises(KeyError):
        registry.param("missing")
    hint = ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")
    hinted = ManagedParamRegistry.from_module(module, shard_hints={"0.weight": hint})
    assert hinted.param("0.weight").shard_hint == hint and hinted.param("0.bias").shard_hint == ParamShardHint()
    with pytest.raises(ValueError, match="unknown parameters"):
        ManagedParamRegistry.from_module(nn.Linear(4, 3), shard_hints={"missing": ParamShardHint()})

    module = nn.Sequential(nn.Linear(4, 6), nn.Linear(6, 2))
    for name, bad, message in [
        ("0.bias", ParamShardHint(split_granularity="matrix_owner"), "matrix_owner"),
        ("0.weight", ParamShardHint(split_granularity="row_block", block_shape=(2, 5)), "second dim"),
        ("0.weight", ParamShardHint(split_granularity="row_block", block_shape=(4, 4)), "not divisible"),
        ("0.weight", ParamShardHint(split_granularity="matrix_owner", block_shape=(2, 4)), "does not accept block_shape"),
        ("0.weight", ParamShardHint(split_granularity="matrix_owner", runtime_kind=ParamRuntimeKind.EXPERT_OWNER), "requires expert_group_id"),
        ("0.weight", ParamShardHint(parallel_role="unknown"), "unknown parallel_role"),
        ("0.weight", ParamShardHint(split_granularity="diagonal"), "unknown split_granularity"),
        ("0.weight", ParamShardHint(runtime_kind="elsewhere"), "unknown runtime_kind"),
        ("0.bias", ParamShardHint(split_granularity="block", block_shape=(4,)), "not divisible"),
        ("0.bias", ParamShardHint(split_granularity="block"), "expects a 1D block_shape"),
        ("0.bias", ParamShardHint(split_granularity="row_block", block_shape=(1,)), "expects a 2D tensor"),
        ("0.weight", ParamShardHint(split_granularity="block", block_shape=(0,)), "must be positive"),
        ("0.weight", ParamShardHint(owner_rank=-1), "owner_rank must be non-negative"),
    ]:
        with pytest.raises(ValueError, match=message):
            ManagedParamRegistry.from_module(module, shard_hints={name: bad})
