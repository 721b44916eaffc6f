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


class ParamRuntimeKind:
    """How the runtime treats a parameter (matrix_fsdp/core/managed_param.py:10-13);
    only the names are used here -- ``EXPERT_OWNER`` keeps an expert's
    parameters on one rank in the expert planner."""

    FSDP_GATHER = "fsdp_gather"
    EP_LOCAL_FSDP = "ep_local_fsdp"
    EXPERT_OWNER = "expert_owner"


_SPLIT_GRANULARITIES = (None, "parameter", "matrix_owner", "row_block", "block")
_RUNTIME_KINDS = (None, ParamRuntimeKind.FSDP_GATHER, ParamRuntimeKind.EP_LOCAL_FSDP, ParamRuntimeKind.EXPERT_OWNER)
_PARALLEL_ROLES = (None, "dense", "embedding", "norm", "router", "routed_expert", "shared_expert")


def _choices(values) -> str:
    return ", ".join(repr(v) for v in sorted(values, key=str))


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


def validate_param_shard_hint(fqn: str, shape, numel: int, hint: ParamShardHint) -> None:
    """A hint must name known vocabulary and fit the tensor it is attached to
    (matrix_fsdp/core/managed_param.py:131-213): whole-parameter granularities
    take no ``block_shape`` (``matrix_owner`` wants a matrix), ``block`` wants
    one size that divides the element count, ``row_block`` a matrix whose rows
    the block divides (a second entry must equal the column count)."""
    shape = tuple(shape)
    if hint.split_granularity not in _SPLIT_GRANULARITIES:
        raise ValueError(f"Param {fqn} has unknown split_granularity={hint.split_granularity!r}; expected {_choices(_SPLIT_GRANULARITIES)}.")
    if hint.runtime_kind not in _RUNTIME_KINDS:
        raise ValueError(f"Param {fqn} has unknown runtime_kind={hint.runtime_kind!r}; expected {_choices(_RUNTIME_KINDS)}.")
    if hint.parallel_role not in _PARALLEL_ROLES:
        raise ValueError(f"Param {fqn} has unknown parallel_role={hint.parallel_role!r}; expected {_choices(_PARALLEL_ROLES)}.")
    if hint.expert_id is not None and hint.expert_id < 0:
        raise ValueError(f"Param {fqn} expert_id must be non-negative, got {hint.expert_id}.")
    if hint.owner_rank is not None and hint.owner_rank < 0:
        raise ValueError(f"Param {fqn} owner_rank must be non-negative, got {hint.owner_rank}.")
    if any(rank < 0 for rank in hint.owner_replica_ranks):
        raise ValueError(f"Param {fqn} owner_replica_ranks must be non-negative, got {hint.owner_replica_ranks}.")
    if hint.runtime_kind == ParamRuntimeKind.EXPERT_OWNER and not hint.expert_group_id:
        raise ValueError(f"Param {fqn} runtime_kind='expert_owner' requires expert_group_id metadata.")
    block = hint.block_shape
    if block is not None:
        if not block:
            raise ValueError(f"Param {fqn} block_shape cannot be empty.")
        if any(dim <= 0 for dim in block):
            raise ValueError(f"Param {fqn} block_shape dims must be positive, got {block}.")
    if hint.split_granularity in (None, "parameter", "matrix_owner"):
        if block is not None:
            raise ValueError(f"Param {fqn} split_granularity={hint.split_granularity!r} does not accept block_shape.")
        if hint.split_granularity == "matrix_owner" and len(shape) != 2:
            raise ValueError(f"Param {fqn} matrix_owner split_granularity expects a 2D tensor, got shape={shape}.")
    elif hint.split_granularity == "block":
        if block is None or len(block) != 1:
            raise ValueError(f"Param {fqn} block split_granularity expects a 1D block_shape.")
        if numel % block[0]:
            raise ValueError(f"Param {fqn} numel={numel} is not divisible by block_shape={block}.")
    else:  # row_block
        if len(shape) != 2:
            raise ValueError(f"Param {fqn} row_block split_granularity expects a 2D tensor, got shape={shape}.")
        if block is None or len(block) not in (1, 2):
            raise ValueError(f"Param {fqn} row_block split_granularity expects a 1D or 2D block_shape.")
        rows, cols = shape
        if len(block) == 2 and block[1] != cols:
            raise ValueError(f"Param {fqn} row_block block_shape second dim={block[1]} must match cols={cols}.")
        if rows % block[0]:
            raise ValueError(f"Param {fqn} rows={rows} is not divisible by row block={block[0]}.")


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
        hint = hints.pop(fqn, None) or ParamShardHint()
        validate_param_shard_hint(fqn, param.shape, n, hint)
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
                shard_hint=hint,
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


@dataclass(frozen=True)
class ManagedParamRegistry:
    """The records of one flat buffer as a read-only sequence with lookup by
    name (matrix_fsdp/core/managed_param.py:46-128)."""

    params: tuple[ManagedParam, ...]

    def __post_init__(self) -> None:
        object.__setattr__(self, "params", tuple(self.params))
        names = [p.fqn for p in self.params]
        if len(set(names)) != len(names):
            raise ValueError("Duplicate managed parameter fqn in registry.")

    def __iter__(self):
        return iter(self.params)

    def __len__(self) -> int:
        return len(self.params)

    def __getitem__(self, index: int) -> ManagedParam:
        return self.params[index]

    @property
    def total_numel(self) -> int:
        return self.params[-1].end if self.params else 0

    @property
    def fqns(self) -> tuple[str, ...]:
        return tuple(p.fqn for p in self.params)

    def param(self, fqn: str) -> ManagedParam:
        for record in self.params:
            if record.fqn == fqn:
                return record
        raise KeyError(fqn)

    def as_list(self) -> list[ManagedParam]:
        return list(self.params)

    @classmethod
    def from_module(cls, module: nn.Module, *, shard_hints: Mapping[str, ParamShardHint] | None = None, ignored_params: set[nn.Parameter] | None = None) -> "ManagedParamRegistry":
        return cls(managed_params_from_module(module, shard_hints=shard_hints, ignored_params=ignored_params))
