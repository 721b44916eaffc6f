"""Owner planners and shard-hint rules against the expectations the reference's own tests hold
(test/fsdp/test_auto_planner.py:417-510 on its ``_SplitQKVLikeBlock(hidden=16, intermediate=64)`` module)."""
import pytest
import torch
from torch import nn

from matrix_fsdp_amd import validate_shard_plan
from matrix_fsdp_amd.core.managed_param import ParamShardHint, managed_params_from_module
from matrix_fsdp_amd.planning import (
    MuonOwnerPlanner,
    ShardHintRule,
    build_shard_hints,
    load_balanced_matrix_owner_tail_group_plans,
    load_balanced_matrix_owner_tail_plan,
    ordered_matrix_owner_tail_plan,
    owner_ranks,
)


class SplitMLP(nn.Module):
    def __init__(self, hidden: int, intermediate: int) -> None:
        super().__init__()
        self.up0 = nn.Linear(hidden, intermediate // 2, bias=False)
        self.up1 = nn.Linear(hidden, intermediate // 2, bias=False)
        self.down = nn.Linear(intermediate // 2, hidden, bias=False)


class SplitQKVBlock(nn.Module):
    """q, k, v, proj 16x16; up0, up1 32x16; down 16x32; two LayerNorms of 16."""

    def __init__(self, hidden: int = 16, intermediate: int = 64) -> None:
        super().__init__()
        self.q = nn.Linear(hidden, hidden, bias=False)
        self.k = nn.Linear(hidden, hidden, bias=False)
        self.v = nn.Linear(hidden, hidden, bias=False)
        self.proj = nn.Linear(hidden, hidden, bias=False)
        self.mlp = SplitMLP(hidden, intermediate)
        self.norm1 = nn.LayerNorm(hidden)
        self.norm2 = nn.LayerNorm(hidden)


@pytest.fixture
def block_params():
    params = list(managed_params_from_module(SplitQKVBlock()))
    return params, {p.fqn: p for p in params}


def test_ordered_plan_maps_matrices_in_module_order_and_the_tail_behind_them(block_params):
    params, by = block_params
    plan = ordered_matrix_owner_tail_plan(params, 8)
    validate_shard_plan(plan)
    want = {"q.weight": 0, "k.weight": 1, "v.weight": 2, "proj.weight": 3, "mlp.up0.weight": 4, "mlp.up1.weight": 5, "mlp.down.weight": 6,
            "norm1.weight": 7, "norm1.bias": 7, "norm2.weight": 7, "norm2.bias": 7}
    assert {fqn: owner_ranks(plan, p) for fqn, p in by.items()} == {fqn: (r,) for fqn, r in want.items()}
    # more matrices than ranks: owners wrap around, the tail goes to the last rank
    small = ordered_matrix_owner_tail_plan(params, 4)
    assert owner_ranks(small, by["mlp.up0.weight"]) == (0,) and owner_ranks(small, by["norm2.bias"]) == (3,)


def test_load_balanced_plan_gives_roles_to_the_lightest_ranks(block_params):
    params, by = block_params
    plan = load_balanced_matrix_owner_tail_plan(params, 8, initial_rank_units=(0, 0, 0, 1024, 1024, 0, 0, 0))
    validate_shard_plan(plan)
    assert owner_ranks(plan, by["mlp.up0.weight"]) == (0,)
    assert owner_ranks(plan, by["mlp.up1.weight"]) == (1,)
    assert owner_ranks(plan, by["mlp.down.weight"]) == (2,)
    assert owner_ranks(plan, by["q.weight"]) == (5,)
    assert owner_ranks(plan, by["norm1.weight"]) == (6,)
    assert plan.shard_sizes == (512, 512, 512, 0, 0, 512, 320, 256)
    assert tuple(seg.numel for seg in plan.rank_segments[6]) == (256, 16, 16, 16, 16)
    with pytest.raises(ValueError, match="initial_rank_units"):
        load_balanced_matrix_owner_tail_plan(params, 8, initial_rank_units=(0, 0))


def test_adjacent_segments_merge_without_merging_owners(block_params):
    params, by = block_params
    plan = load_balanced_matrix_owner_tail_plan(params, 4, merge_adjacent_rank_segments=True)
    validate_shard_plan(plan)
    assert owner_ranks(plan, by["q.weight"]) == (3,) and owner_ranks(plan, by["k.weight"]) == (3,)
    assert owner_ranks(plan, by["norm1.weight"]) == (2,)
    assert tuple(seg.numel for seg in plan.rank_segments[3]) == (512,)
    assert tuple(seg.numel for seg in plan.rank_segments[2]) == (576,)


def test_group_plans_balance_across_units(block_params):
    params, by = block_params
    plans = load_balanced_matrix_owner_tail_group_plans((params, params, params, params), 8)
    assert tuple(sum(plan.shard_sizes[r] for plan in plans) for r in range(8)) == (1344, 1344, 1344, 1344, 1280, 1280, 1280, 1280)
    assert [owner_ranks(plan, by["mlp.up0.weight"]) for plan in plans] == [(0,), (3,), (6,), (1,)]


def test_muon_owner_planner_is_role_greedy_across_calls(block_params):
    params, by = block_params
    planner = MuonOwnerPlanner()
    plans = [planner(params, 8) for _ in range(4)]
    assert owner_ranks(plans[0], by["mlp.up0.weight"]) == (0,)
    assert owner_ranks(plans[0], by["q.weight"]) == (3,)
    assert owner_ranks(plans[0], by["norm1.weight"]) == (7,)
    assert owner_ranks(plans[1], by["mlp.up0.weight"]) == (7,)
    assert owner_ranks(plans[1], by["q.weight"]) == (5,)
    assert tuple(sum(plan.shard_sizes[r] for plan in plans) for r in range(8)) == (1536, 1280, 1152, 1280, 1344, 1280, 1280, 1344)


def test_owner_rank_hint_pins_a_role_and_conflicts_are_rejected():
    module = nn.Sequential(nn.Linear(4, 4, bias=False), nn.Linear(4, 4, bias=False))
    params = list(managed_params_from_module(module, shard_hints={"0.weight": ParamShardHint(owner_rank=3)}))
    plan = load_balanced_matrix_owner_tail_group_plans((params,), 4)[0]
    assert owner_ranks(plan, params[0]) == (3,) and owner_ranks(plan, params[1]) == (0,)
    with pytest.raises(ValueError, match=r"owner_rank=3 must be in \[0, 2\)"):
        load_balanced_matrix_owner_tail_group_plans((params,), 2)


def test_default_shard_hint_rules():
    class Model(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.embed = nn.Embedding(10, 4)
            self.block = SplitQKVBlock(4, 8)
            self.head = nn.Linear(4, 10, bias=True)
            self.scale = nn.Parameter(torch.ones(4))
            self.table = nn.Parameter(torch.zeros(3, 4))

    hints = build_shard_hints(Model())
    muon = ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")
    adamw = ParamShardHint(optimizer_type="adamw", split_granularity="parameter")
    assert hints["block.q.weight"] == muon and hints["head.weight"] == muon
    assert hints["embed.weight"] == adamw and hints["block.norm1.weight"] == adamw and hints["head.bias"] == adamw and hints["scale"] == adamw
    assert "table" not in hints  # a bare 2-D parameter matches no rule
    custom = build_shard_hints(Model(), rules=[ShardHintRule("all", lambda fqn, owner, name, p: adamw)], overrides={"table": muon})
    assert custom["block.q.weight"] == adamw and custom["table"] == muon
    with pytest.raises(ValueError, match="unknown parameters: nope"):
        build_shard_hints(Model(), overrides={"nope": muon})


def test_moe_hint_rules_and_expert_planner():
    """test/fsdp/test_shard_hint.py:68-110: rule names in order, experts and router recognised by module path; the
    hinted experts then stay together under ``expert_owner_tail_plan`` and pass the layout validator."""
    from matrix_fsdp_amd.core.managed_param import ManagedParamRegistry, ParamRuntimeKind
    from matrix_fsdp_amd.planning import default_shard_hint_rules, expert_owner_tail_plan, validate_group_layout

    assert tuple(rule.name for rule in default_shard_hint_rules()) == (
        "moe_expert_owner", "router", "muon_linear_weight", "no_split_embedding", "no_split_norm", "no_split_bias", "no_split_1d",
    )

    class Expert(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.w1 = nn.Linear(4, 8, bias=True)
            self.w2 = nn.Linear(8, 4, bias=False)

    class MoEBlock(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.router = nn.Linear(4, 2, bias=False)
            self.experts = nn.ModuleList([Expert(), Expert(), Expert()])
            self.norm = nn.LayerNorm(4)

    class Model(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.moe = MoEBlock()
            self.experts = nn.Linear(4, 4)  # no expert index below it: an ordinary linear layer

    model = Model()
    hints = build_shard_hints(model)
    assert hints["moe.experts.0.w1.weight"] == ParamShardHint(
        optimizer_type="muon", split_granularity="matrix_owner", runtime_kind=ParamRuntimeKind.EXPERT_OWNER, parallel_role="routed_expert", expert_id=0, expert_group_id="moe.experts.0"
    )
    assert hints["moe.experts.0.w1.bias"] == ParamShardHint(
        optimizer_type="adamw", split_granularity="parameter", runtime_kind=ParamRuntimeKind.EXPERT_OWNER, parallel_role="routed_expert", expert_id=0, expert_group_id="moe.experts.0"
    )
    assert hints["moe.experts.1.w2.weight"].expert_group_id == "moe.experts.1" and hints["moe.experts.2.w2.weight"].expert_id == 2
    assert hints["moe.router.weight"] == ParamShardHint(optimizer_type="adamw", split_granularity="parameter", runtime_kind=ParamRuntimeKind.FSDP_GATHER, parallel_role="router")
    assert hints["experts.weight"] == ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")
    assert hints["moe.norm.weight"] == ParamShardHint(optimizer_type="adamw", split_granularity="parameter")

    params = ManagedParamRegistry.from_module(model, shard_hints=hints).as_list()
    layout = expert_owner_tail_plan(params, 2)
    validate_group_layout(layout, params, 2)  # includes: one owner rank per expert group
    owners = {group: {layout.owner_ranks(p.fqn) for p in params if p.shard_hint.expert_group_id == group} for group in ("moe.experts.0", "moe.experts.1", "moe.experts.2")}
    assert all(len(ranks) == 1 for ranks in owners.values())
    # three experts of 72 elements: ranks 0, 1, 0; the dense tail (16 + 8 + 4 + 4 + 4), largest first, all fits on rank 1
    assert layout.shard_sizes == (144, 108)
    assert layout.owner_ranks("moe.experts.2.w1.bias") == (0,) and layout.owner_ranks("moe.router.weight") == (1,)
