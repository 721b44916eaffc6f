"""Metadata producers for whole-parameter owner layouts and shard hints."""
from .owner_plans import (
    MuonOwnerPlanner,
    load_balanced_matrix_owner_tail_group_plans,
    load_balanced_matrix_owner_tail_plan,
    ordered_matrix_owner_tail_plan,
    owner_ranks,
    whole_param_assignment_plan,
)
from .shard_hint import ShardHintRule, build_shard_hints, default_shard_hint_rules

__all__ = [
    "MuonOwnerPlanner",
    "load_balanced_matrix_owner_tail_group_plans",
    "load_balanced_matrix_owner_tail_plan",
    "ordered_matrix_owner_tail_plan",
    "owner_ranks",
    "whole_param_assignment_plan",
    "ShardHintRule",
    "build_shard_hints",
    "default_shard_hint_rules",
]
