"""``fully_shard`` / ``matrix_fully_shard``: wrap a module's parameters into one flat-buffer unit.

The entry points keep the reference's names and the arguments that matter on a
single device (matrix_fsdp/api.py:213-263 ``fully_shard``, :266-330
``matrix_fully_shard``).  There is no process group here: ``world_size`` and
``rank`` say which simulated world the unit is sharded for (default: a world
of one, the reference's single-rank path).  Arguments that only steer
collectives, prefetching, offload or the planner families are not accepted.
"""
from __future__ import annotations

from dataclasses import dataclass
from functools import partial
from typing import Callable, Mapping

import torch
from torch import nn
from torch.distributed.fsdp import OffloadPolicy
from torch.distributed.tensor import Shard

from .core.layout import ShardPlan
from .core.managed_param import ManagedParam, ParamShardHint
from .planning.group_plans import hinted_ordered_group_plan
from .planning.owner_plans import MuonOwnerPlanner
from .planning.shard_hint import build_shard_hints
from .policy.wrap import WrapPolicy
from .runtime.param_group import MatrixFSDPParamGroup

# optimizer_policy values of fully_shard (matrix_fsdp/api.py:43-54)
_MUON_OPTIMIZER_POLICIES = {"mixed_muon_adamw", "muon_adamw", "muon_shard_aware", "muon"}
_NOOP_OPTIMIZER_POLICIES = {"default", "none", "adamw", "sgd"}


# arguments of the reference's matrix_fully_shard (matrix_fsdp/api.py:266-300) that choose collectives, their
# scheduling or tracing: nothing for them to steer without a process group
_SINGLE_DEVICE_NOOPS = frozenset(
    {
        "dp_mesh_dims",
        "dp_shard_mesh_dim",
        "dp_replicate_mesh_dim",
        "forward_prefetch",
        "backward_prefetch",
        "param_gather_strategy",
        "matrix_collective_backend",
        "grad_reduce_strategy",
        "backward_reduce_strategy",
        "runtime_layout_policy",
        "runtime_trace_enabled",
        "shrink_full_param_storage_after_backward",
    }
)


@dataclass(frozen=True)
class MixedPrecisionPolicy:
    """Field-compatible with ``torch.distributed.fsdp.MixedPrecisionPolicy``, which is accepted as well."""

    param_dtype: torch.dtype | None = None
    reduce_dtype: torch.dtype | None = None
    output_dtype: torch.dtype | None = None
    cast_forward_inputs: bool = True


_DEFAULT_MP_POLICY = MixedPrecisionPolicy()


def validate_mixed_precision_policy(mp_policy) -> None:
    for name in ("param_dtype", "reduce_dtype", "output_dtype"):
        dtype = getattr(mp_policy, name, None)
        if dtype is not None and not (isinstance(dtype, torch.dtype) and dtype.is_floating_point):
            raise ValueError(f"mp_policy.{name} must be a floating-point torch.dtype or None, got {dtype!r}.")


def matrix_fully_shard(
    module: nn.Module,
    *,
    world_size: int = 1,
    rank: int = 0,
    planner: Callable[[list[ManagedParam], int], ShardPlan] | None = None,
    shard_hints: Mapping[str, ParamShardHint] | None = None,
    ignored_params: set[nn.Parameter] | None = None,
    reshard_after_forward: bool = True,
    mp_policy=_DEFAULT_MP_POLICY,
    wrap_policy: WrapPolicy | None = None,
    auto_shard_hints: bool = False,
    auto_planner_policy: str | None = None,
    use_saved_tensor_hooks: bool = True,
    full_param_buffer_pool=None,
    use_zero_copy_grad_bucket: bool = False,
    mesh=None,
    group_planner: Callable[[list[ManagedParam], int], ShardPlan] | None = None,
    offload_policy=None,
    finalize_after_backward: bool = True,
    **single_device_noops,
) -> nn.Module:
    """Turns ``module`` into one unit: its parameters (those no nested unit
    manages yet) move into a flat buffer sharded by ``planner`` for the
    simulated world, become views of rank ``rank``'s local shard, and forward /
    backward hooks unshard and reshard them.  Returns ``module``.

    With ``wrap_policy`` the module tree is walked from the top: a module the
    policy selects becomes a unit (and is not descended into), the others'
    own parameters stay unmanaged (matrix_fsdp/api.py:309-378, 505-624).
    ``auto_shard_hints`` derives the hints from the module structure;
    ``auto_planner_policy="muon_shard_aware"`` keeps every parameter whole on
    an owner rank (the other planner families of the reference do not exist
    here).  ``use_saved_tensor_hooks`` (default on, as in the reference) keeps
    autograd from pinning a unit's full buffer between forward and backward;
    ``full_param_buffer_pool`` (a ``FullParamBufferPool``) lets units of equal
    size unshard into the same storage; ``use_zero_copy_grad_bucket`` (default
    off, as in the reference) lets autograd write gradients straight into the
    reduce-scatter workspace where the layout and dtypes allow it.

    Of the reference's further arguments, ``group_planner`` is ``planner``
    under its other name; ``mesh`` (one rank at most), ``offload_policy`` (no
    offload) and ``finalize_after_backward`` (``True``) are taken in their
    neutral values; the switches that only choose collectives or the order in
    which they are issued (``_SINGLE_DEVICE_NOOPS``) are accepted and have no
    effect on one device.  Anything else is a ``TypeError``."""
    unknown = set(single_device_noops) - _SINGLE_DEVICE_NOOPS
    if unknown:
        raise TypeError(f"matrix_fully_shard() got unexpected keyword arguments: {', '.join(sorted(unknown))}.")
    _refuse_multi_device_arguments(mesh, offload_policy, single_device_noops.get("dp_mesh_dims"))
    if any(single_device_noops.get(name) is not None for name in ("dp_shard_mesh_dim", "dp_replicate_mesh_dim")):
        raise NotImplementedError("dp_shard_mesh_dim / dp_replicate_mesh_dim select dimensions of a multi-rank mesh, which does not exist here.")
    if not finalize_after_backward:
        raise NotImplementedError("finalize_after_backward=False leaves the reduce to the caller; units here always finalise at the end of the backward.")
    if group_planner is not None:
        if planner is not None:
            raise ValueError("Pass either planner or group_planner, not both.")
        planner = group_planner
    validate_mixed_precision_policy(mp_policy)
    if not isinstance(reshard_after_forward, bool):
        # an int asks for resharding to a smaller world after forward (matrix_fsdp/runtime/fsdp_unit.py:1705-1720)
        raise NotImplementedError("reshard_after_forward=int requires post-forward subgroup resharding, which does not exist here; pass a bool.")
    if auto_planner_policy is not None:
        if str(auto_planner_policy).lower() != "muon_shard_aware":
            raise ValueError(f"auto_planner_policy={auto_planner_policy!r} is not available; only 'muon_shard_aware' is.")
        if planner is not None:
            raise ValueError("Pass either auto_planner_policy or an explicit planner, not both.")
        planner = MuonOwnerPlanner()  # one object for every unit of this call: ranks are balanced across the units
    unit_args = dict(
        world_size=world_size,
        rank=rank,
        planner=planner,
        ignored_params=ignored_params,
        reshard_after_forward=reshard_after_forward,
        param_dtype=getattr(mp_policy, "param_dtype", None),
        reduce_dtype=getattr(mp_policy, "reduce_dtype", None),
        output_dtype=getattr(mp_policy, "output_dtype", None),
        cast_forward_inputs=getattr(mp_policy, "cast_forward_inputs", True),
        use_saved_tensor_hooks=use_saved_tensor_hooks,
        full_param_buffer_pool=full_param_buffer_pool,
        use_zero_copy_grad_bucket=use_zero_copy_grad_bucket,
    )
    if wrap_policy is not None:
        if shard_hints is not None:
            raise ValueError("wrap_policy does not support explicit shard_hints yet.")
        if _wrap_selected(module, wrap_policy, ignored_params, auto_shard_hints, unit_args) == 0:
            raise ValueError("wrap_policy did not select any modules to shard.")
        return module
    _make_unit(module, shard_hints, ignored_params, auto_shard_hints, unit_args)
    return module


def _own_hints(module: nn.Module, ignored_params: set[nn.Parameter] | None) -> dict[str, ParamShardHint]:
    """Structure-derived hints for the parameters this unit will manage."""
    skip = {id(p) for p in ignored_params or ()}
    mine = {fqn for fqn, p in module.named_parameters() if id(p) not in skip and not getattr(p, "_matrix_fsdp_managed", False)}
    return {fqn: hint for fqn, hint in build_shard_hints(module).items() if fqn in mine}


def _make_unit(module, shard_hints, ignored_params, auto_shard_hints: bool, unit_args: dict) -> None:
    if getattr(module, "_matrix_fsdp_param_group", None) is not None:
        raise ValueError("module is already wrapped by matrix_fully_shard().")
    if auto_shard_hints and shard_hints is None:
        shard_hints = _own_hints(module, ignored_params) or None
    MatrixFSDPParamGroup(module, shard_hints=shard_hints, **unit_args)


def _wrap_selected(module: nn.Module, wrap_policy: WrapPolicy, ignored_params, auto_shard_hints: bool, unit_args: dict) -> int:
    if wrap_policy(module):
        skip = {id(p) for p in ignored_params or ()}
        if not any(id(p) not in skip for p in module.parameters()):
            return 0
        _make_unit(module, None, ignored_params, auto_shard_hints, unit_args)
        return 1
    return sum(_wrap_selected(child, wrap_policy, ignored_params, auto_shard_hints, unit_args) for child in module.children())


def _leading_dim_shard_hint(fqn: str, param: nn.Parameter) -> ParamShardHint:
    """``Shard(0)`` as a hint: a matrix may be cut between any two rows, any other
    tensor between any two slices along its first dimension (matrix_fsdp/api.py:159-167)."""
    if param.ndim == 0:
        raise NotImplementedError(f"MatrixFSDP cannot apply Shard(0) to scalar parameter {fqn}.")
    if param.ndim == 2:
        return ParamShardHint(split_granularity="row_block", block_shape=(1, int(param.shape[1])))
    return ParamShardHint(split_granularity="block", block_shape=(int(param.numel() // param.shape[0]),))


def _refuse_multi_device_arguments(mesh, offload_policy, dp_mesh_dims) -> None:
    """The reference's arguments for process meshes and host offload are taken
    in their neutral values only: there is one device and no process group."""
    if mesh is not None and int(mesh.size()) != 1:
        raise NotImplementedError(
            "fully_shard(mesh=...) over several ranks needs a process group, which does not exist here; "
            "world_size= / rank= shard a unit for a simulated world on the one device."
        )
    if dp_mesh_dims is not None:
        raise NotImplementedError("fully_shard(dp_mesh_dims=...) selects dimensions of a multi-rank mesh, which does not exist here.")
    if offload_policy is not None:
        # torch.distributed.fsdp.OffloadPolicy() means "no offload"; CPUOffloadPolicy on a device-resident model is
        # refused by the reference as well (matrix_fsdp/core/mixed_precision.py:39-56)
        if not isinstance(offload_policy, OffloadPolicy):
            raise TypeError(f"offload_policy must be an OffloadPolicy, got {type(offload_policy).__name__}.")
        if type(offload_policy) is not OffloadPolicy:
            raise NotImplementedError(f"fully_shard(offload_policy={type(offload_policy).__name__}) is not available: shards stay in device memory.")


def fully_shard(
    module: nn.Module,
    *,
    mesh=None,
    reshard_after_forward: bool | None = None,
    shard_placement_fn: Callable[[nn.Parameter], object | None] | None = None,
    mp_policy=_DEFAULT_MP_POLICY,
    offload_policy=None,
    ignored_params: set[nn.Parameter] | None = None,
    dp_mesh_dims=None,
    optimizer_policy: str | None = None,
    world_size: int = 1,
    rank: int = 0,
    planner: Callable[[list[ManagedParam], int], ShardPlan] | None = None,
) -> nn.Module:
    """FSDP2-style spelling (matrix_fsdp/api.py:213-263): ``shard_placement_fn``
    maps a parameter to ``torch.distributed.tensor.Shard(0)`` or ``None`` (a
    ``ParamShardHint`` is accepted as well); parameters placed with ``Shard(0)``
    may be cut between rows (first-dimension slices) and the unit's flat buffer
    is then cut rank-contiguously at such boundaries (``hinted_ordered_group_plan``);
    ``reshard_after_forward`` defaults to ``True``.  A Muon ``optimizer_policy`` (``"muon"``,
    ``"mixed_muon_adamw"``, ...) derives the hints from the module structure
    (``build_shard_hints``) and keeps every parameter whole on an owner rank
    (``MuonOwnerPlanner``; pass one planner object to all units to balance the
    ranks across units).  The first nine parameters are the reference's, in its
    order; ``mesh`` (a one-rank mesh at most), ``offload_policy`` (no offload)
    and ``dp_mesh_dims`` (``None``) are accepted in their neutral values, and
    ``world_size`` / ``rank`` / ``planner`` are this build's additions."""
    _refuse_multi_device_arguments(mesh, offload_policy, dp_mesh_dims)
    hints: dict[str, ParamShardHint] = {}
    if optimizer_policy is not None:
        policy = optimizer_policy.lower()
        if policy in _MUON_OPTIMIZER_POLICIES:
            if shard_placement_fn is not None:
                raise ValueError("fully_shard optimizer_policy cannot be combined with shard_placement_fn.")
            hints = _own_hints(module, ignored_params)
            planner = planner or MuonOwnerPlanner()
        elif policy not in _NOOP_OPTIMIZER_POLICIES:
            allowed = sorted(_MUON_OPTIMIZER_POLICIES | _NOOP_OPTIMIZER_POLICIES)
            raise ValueError(f"Unknown fully_shard optimizer_policy={optimizer_policy!r}; expected one of {allowed}.")
    if shard_placement_fn is not None:
        ignored = {id(p) for p in ignored_params or ()}
        placed = False
        for fqn, param in module.named_parameters():
            if id(param) in ignored or getattr(param, "_matrix_fsdp_managed", False):
                continue
            placement = shard_placement_fn(param)
            if placement is None:
                continue
            if isinstance(placement, ParamShardHint):  # an explicit hint is taken as it is
                hints[fqn] = placement
                continue
            if not isinstance(placement, Shard):
                raise NotImplementedError(
                    "MatrixFSDP fully_shard shard_placement_fn currently supports only None or torch.distributed.tensor.Shard placements."
                )
            if placement.dim != 0:
                raise NotImplementedError(
                    "MatrixFSDP fully_shard shard_placement_fn currently supports only Shard(0). Sharding non-leading tensor "
                    "dimensions would require non-contiguous local storage segments."
                )
            hints[fqn] = _leading_dim_shard_hint(fqn, param)
            placed = True
        if placed and planner is None:
            # rank-contiguous cut of the flat buffer at the hinted boundaries (matrix_fsdp/api.py:153-156)
            planner = partial(hinted_ordered_group_plan, default_granularity="parameter")
    return matrix_fully_shard(
        module,
        world_size=world_size,
        rank=rank,
        planner=planner,
        shard_hints=hints or None,
        ignored_params=ignored_params,
        reshard_after_forward=True if reshard_after_forward is None else reshard_after_forward,
        mp_policy=mp_policy,
    )
