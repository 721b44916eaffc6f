"""Per-parameter records of a flat buffer.

``ManagedParam`` carries the same fields as the reference's record
(matrix_fsdp/core/managed_param.py:29-44): a parameter occupies
``[offset, end)`` of the flat buffer, offsets being assigned in
``named_parameters`` order (matrix_fsdp/core/managed_param.py:103-123).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable, Mapping

import torch
from torch import nn


@dataclass(frozen=True)
class ParamShardHint:
    """Planner/optimizer hints attached to a parameter
    (matrix_fsdp/core/managed_param.py:16-26).  Only ``optimizer_type`` and
    ``owner_rank`` are read on the copy / optimizer path."""

    optimizer_type: str | None = None
    split_granularity: str | None = None
    block_shape: tuple[int, ...] | None = None
    runtime_kind: str | None = None
    parallel_role: str | None = None
    expert_id: int | None = None
    expert_group_id: str | None = None
    owner_rank: int | None = None
    owner_replica_ranks: tuple[int, ...] = ()


@dataclass
class ManagedParam:
    fqn: str
    param: nn.Parameter
    shape: torch.Size
    dtype: torch.dtype
    device: torch.device
    numel: int
    offset: int
    end: int
    shard_hint: ParamShardHint = field(default_factory=ParamShardHint)

    @property
    def local_name(self) -> str:
        return self.fqn.rsplit(".", 1)[-1]


def managed_params_from_named(
    named_params: Iterable[tuple[str, nn.Parameter]],
    *,
    shard_hints: Mapping[str, ParamShardHint] | None = None,
) -> tuple[ManagedParam, ...]:
    """Assigns flat offsets in iteration order; duplicate names are an error
    (matrix_fsdp/core/managed_param.py:52-58)."""
    hints = dict(shard_hints or {})
    records: list[ManagedParam] = []
    seen: set[str] = set()
    cursor = 0
    for fqn, param in named_params:
        if fqn in seen:
            raise ValueError(f"Duplicate managed parameter fqn: {fqn}.")
        seen.add(fqn)
        n = param.numel()
        records.append(
            ManagedParam(
                fqn=fqn,
                param=param,
                shape=param.shape,
                dtype=param.dtype,
                device=param.device,
                numel=n,
                offset=cursor,
                end=cursor + n,
                shard_hint=hints.pop(fqn, ParamShardHint()),
            )
        )
        cursor += n
    if hints:
        raise ValueError(f"Shard hints refer to unknown parameters: {', '.join(sorted(hints))}.")
    return tuple(records)


def managed_params_from_module(
    module: nn.Module,
    *,
    shard_hints: Mapping[str, ParamShardHint] | None = None,
    ignored_params: set[nn.Parameter] | None = None,
) -> tuple[ManagedParam, ...]:
    """``named_parameters`` order, shared parameters rejected
    (matrix_fsdp/core/managed_param.py:79-101)."""
    ignored = {id(p) for p in ignored_params or ()}
    aliases: dict[int, list[str]] = {}
    for fqn, param in module.named_parameters(recurse=True, remove_duplicate=False):
        if id(param) not in ignored:
            aliases.setdefault(id(param), []).append(fqn)
    shared = [names for names in aliases.values() if len(names) > 1]
    if shared:
        raise NotImplementedError(
            "MatrixFSDP does not support shared parameters yet. Shared parameter aliases: "
            + "; ".join(",".join(names) for names in shared)
            + "."
        )
    named = [(fqn, p) for fqn, p in module.named_parameters(recurse=True) if id(p) not in ignored]
    return managed_params_from_named(named, shard_hints=shard_hints)
