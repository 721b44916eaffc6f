"""Shard hints from module structure (matrix_fsdp/planning/shard_hint.py:15-160).

A rule looks at one parameter -- its name, the module that owns it -- and
either returns a ``ParamShardHint`` or passes; the first rule that answers
wins.  The default rules put Muon on the weights of ``nn.Linear`` (kept whole
on an owner rank) and AdamW on embeddings, normalisation layers, biases and
every other vector (never cut inside a parameter).  Ahead of them go the
mixture-of-experts rules: every parameter under ``<...>.experts.<n>.`` belongs
to expert ``n`` of that group and must stay with its expert's owner rank
(``runtime_kind="expert_owner"``, what ``expert_owner_tail_plan`` groups by),
and parameters of a ``gate`` / ``router`` module are gathered AdamW parameters.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Mapping, Sequence

from torch import nn

from ..core.managed_param import ParamRuntimeKind, ParamShardHint

ShardHintRuleFn = Callable[[str, nn.Module, str, nn.Parameter], "ParamShardHint | None"]

_NORM_TYPES = (
    nn.BatchNorm1d,
    nn.BatchNorm2d,
    nn.BatchNorm3d,
    nn.GroupNorm,
    nn.InstanceNorm1d,
    nn.InstanceNorm2d,
    nn.InstanceNorm3d,
    nn.LayerNorm,
)
_WHOLE_ADAMW = ParamShardHint(optimizer_type="adamw", split_granularity="parameter")


@dataclass(frozen=True)
class ShardHintRule:
    name: str
    apply: ShardHintRuleFn


def _expert_of(fqn: str, expert_module_names: Sequence[str]) -> tuple[int, str] | None:
    """``(expert id, group id)`` for ``a.experts.3.w1.weight`` -> ``(3, "a.experts.3")``;
    the expert index must be followed by at least a module and a parameter name
    (shard_hint.py:171-185)."""
    parts = fqn.split(".")
    for i, part in enumerate(parts[:-2]):
        if part in expert_module_names and parts[i + 1].isdigit():
            return int(parts[i + 1]), ".".join(parts[: i + 2])
    return None


def moe_expert_owner_rule(*, expert_module_names: Sequence[str] = ("experts",)) -> ShardHintRule:
    names = tuple(expert_module_names)

    def apply(fqn: str, owner: nn.Module, local: str, param: nn.Parameter) -> ParamShardHint | None:
        found = _expert_of(fqn, names)
        if found is None:
            return None
        matrix = param.ndim == 2
        return ParamShardHint(
            optimizer_type="muon" if matrix else "adamw",
            split_granularity="matrix_owner" if matrix else "parameter",
            runtime_kind=ParamRuntimeKind.EXPERT_OWNER,
            parallel_role="routed_expert",
            expert_id=found[0],
            expert_group_id=found[1],
        )

    return ShardHintRule("moe_expert_owner", apply)


def router_rule(*, module_names: Sequence[str] = ("gate", "router")) -> ShardHintRule:
    names = tuple(module_names)
    hint = ParamShardHint(optimizer_type="adamw", split_granularity="parameter", runtime_kind=ParamRuntimeKind.FSDP_GATHER, parallel_role="router")
    return ShardHintRule("router", lambda fqn, owner, local, p: hint if any(part in names for part in fqn.split(".")[:-1]) else None)


def muon_linear_weight_rule() -> ShardHintRule:
    hint = ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")
    return ShardHintRule("muon_linear_weight", lambda fqn, owner, local, p: hint if isinstance(owner, nn.Linear) and local == "weight" and p.ndim == 2 else None)


def no_split_embedding_rule() -> ShardHintRule:
    return ShardHintRule("no_split_embedding", lambda fqn, owner, local, p: _WHOLE_ADAMW if isinstance(owner, nn.Embedding) and local == "weight" else None)


def no_split_norm_rule() -> ShardHintRule:
    return ShardHintRule("no_split_norm", lambda fqn, owner, local, p: _WHOLE_ADAMW if isinstance(owner, _NORM_TYPES) else None)


def no_split_bias_rule() -> ShardHintRule:
    return ShardHintRule("no_split_bias", lambda fqn, owner, local, p: _WHOLE_ADAMW if local == "bias" else None)


def no_split_1d_rule() -> ShardHintRule:
    return ShardHintRule("no_split_1d", lambda fqn, owner, local, p: _WHOLE_ADAMW if p.ndim <= 1 else None)


def default_shard_hint_rules() -> tuple[ShardHintRule, ...]:
    return (
        moe_expert_owner_rule(),
        router_rule(),
        muon_linear_weight_rule(),
        no_split_embedding_rule(),
        no_split_norm_rule(),
        no_split_bias_rule(),
        no_split_1d_rule(),
    )


def build_shard_hints(
    module: nn.Module,
    *,
    rules: Sequence[ShardHintRule] | None = None,
    overrides: Mapping[str, ParamShardHint] | None = None,
) -> dict[str, ParamShardHint]:
    selected = tuple(rules or default_shard_hint_rules())
    modules = dict(module.named_modules())
    hints: dict[str, ParamShardHint] = {}
    names = []
    for fqn, param in module.named_parameters(recurse=True, remove_duplicate=True):
        names.append(fqn)
        owner_fqn, _, local = fqn.rpartition(".")
        for rule in selected:
            hint = rule.apply(fqn, modules[owner_fqn], local, param)
            if hint is not None:
                hints[fqn] = hint
                break
    if overrides:
        unknown = set(overrides) - set(names)
        if unknown:
            raise ValueError(f"Shard hint overrides refer to unknown parameters: {', '.join(sorted(unknown))}.")
        hints.update(overrides)
    return hints
