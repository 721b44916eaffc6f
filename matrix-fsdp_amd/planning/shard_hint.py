"""Shard hints from module structure (matrix_fsdp/planning/shard_hint.py:15-160).

A rule looks at one parameter -- its name, the module that owns it -- and
either returns a ``ParamShardHint`` or passes; the first rule that answers
wins.  The default rules put Muon on the weights of ``nn.Linear`` (kept whole
on an owner rank) and AdamW on embeddings, normalisation layers, biases and
every other vector (never cut inside a parameter).  The reference's
mixture-of-experts rules (expert owners, routers) are not part of this build.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Mapping, Sequence

from torch import nn

from ..core.managed_param import ParamShardHint

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


def default_shard_hint_rules() -> tuple[ShardHintRule, ...]:
    return (
        ShardHintRule(
            "muon_linear_weight",
            lambda fqn, owner, name, p: ParamShardHint(optimizer_type="muon", split_granularity="matrix_owner")
            if isinstance(owner, nn.Linear) and name == "weight" and p.ndim == 2
            else None,
        ),
        ShardHintRule("no_split_embedding", lambda fqn, owner, name, p: _WHOLE_ADAMW if isinstance(owner, nn.Embedding) and name == "weight" else None),
        ShardHintRule("no_split_norm", lambda fqn, owner, name, p: _WHOLE_ADAMW if isinstance(owner, _NORM_TYPES) else None),
        ShardHintRule("no_split_bias", lambda fqn, owner, name, p: _WHOLE_ADAMW if name == "bias" else None),
        ShardHintRule("no_split_1d", lambda fqn, owner, name, p: _WHOLE_ADAMW if p.ndim <= 1 else None),
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
