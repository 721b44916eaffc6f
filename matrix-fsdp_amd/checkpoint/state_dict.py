"""MatrixFSDP state dicts and their DCP (PyTorch Distributed Checkpoint) form.

What is stored, per unit: the rank's local parameter shard (optionally its
local gradient shard, optionally debug copies of the full parameters) plus a
plain-data description of the layout; per optimizer component: every state
tensor of every local parameter under a key that names component, parameter
and state.  Dict keys, tensor keys and file names are the reference's
(matrix_fsdp/checkpoint/state_dict.py:61-1396), so either side reads the
other's checkpoints of the features both have.

Differences that follow from running on one HIP device:

* There is never a process group.  ``process_group`` / ``no_dist`` are accepted
  for signature compatibility and must describe a single process; the ranks of
  a simulated world are written together by
  ``save_matrix_dcp_simulated_world``, which produces the keys and the
  metadata file a job of that many processes would.
* Loading into a different layout moves data with segment programs: the source
  ranks' shards are read straight into one packed buffer, one launch unpacks it
  to flat-buffer order along the *saved* segments and one launch takes the
  target rank's shard.  Optimizer state rides the same two programs, one flat
  buffer per state name.  Source layouts with several segments per rank are
  therefore handled, which concatenating the source shards
  (state_dict.py:934-939) is not.
* Planner results, layout contracts, collective strategies and offload do not
  exist here; their keys are present and hold ``None`` (or the fixed value
  that describes this runtime).
"""
from __future__ import annotations

from collections.abc import Iterable, Mapping, Sequence
from copy import deepcopy
from math import prod
from os import PathLike
from pathlib import Path
from typing import Any

import torch
from torch import nn

from ..core.layout import LayoutSegment, ShardPlan
from ..kernels import native
from ..kernels.segment_program import CONVERTIBLE, unpack_program
from ..optim.state import MatrixFSDPOptimizerStateManager
from ..runtime.flat_buffer import MatrixFlatBuffer
from ..runtime.param_group import MatrixFSDPParamGroup
from . import dcp_io
from .metadata import (
    canonical,
    dtype_from_string,
    layout_metadata,
    layout_segment_metadata,
    matrix_shard_metadata,
    param_key,
    param_metadata,
)

MATRIX_STATE_DICT_VERSION = 1
MATRIX_DCP_FORMAT_VERSION = 1

UnitRefs = list[tuple[str, MatrixFSDPParamGroup]]


# ---------------------------------------------------------------------------
# units of a module


def collect_param_group_refs(module_or_units) -> UnitRefs:
    """``(module_fqn, unit)`` for every unit that manages parameters: by module
    path for a module, ``unit<i>`` for a bare list of units, ``""`` for one."""
    if isinstance(module_or_units, MatrixFSDPParamGroup):
        return [("", module_or_units)]
    if isinstance(module_or_units, nn.Module):
        refs, seen = [], set()
        for module_fqn, module in module_or_units.named_modules(remove_duplicate=True):
            unit = getattr(module, "_matrix_fsdp_param_group", None)
            if unit is None or id(unit) in seen:
                continue
            if not isinstance(unit, MatrixFSDPParamGroup):
                raise TypeError(f"Expected MatrixFSDPParamGroup, got {type(unit)!r}.")
            seen.add(id(unit))
            if unit.flat_buffer is not None:
                refs.append((module_fqn, unit))
        return refs
    refs = []
    for index, unit in enumerate(module_or_units):
        if not isinstance(unit, MatrixFSDPParamGroup):
            raise TypeError(f"Expected MatrixFSDPParamGroup, got {type(unit)!r}.")
        refs.append((f"unit{index}", unit))
    return refs


def _flat_buffer(unit: MatrixFSDPParamGroup) -> MatrixFlatBuffer:
    if unit.flat_buffer is None:
        raise ValueError("MatrixFSDP checkpointing requires a unit with managed parameters.")
    return unit.flat_buffer


def _unit_states(state: Mapping[str, Any], *, context: str) -> list[dict[str, Any]]:
    units = state.get("param_groups")
    if units is None:
        units = state.get("units")
    if not isinstance(units, list):
        raise TypeError(f"MatrixFSDP {context} must contain a list at key 'param_groups' or legacy key 'units'.")
    return units


def _stored(tensor: torch.Tensor, *, clone: bool) -> torch.Tensor:
    tensor = tensor.detach()
    return tensor.clone() if clone else tensor


# ---------------------------------------------------------------------------
# in-memory state dict


def _unit_state_dict(unit: MatrixFSDPParamGroup, *, unit_index: int, module_fqn: str, include_grads: bool, full_state: bool, clone: bool) -> dict[str, Any]:
    fb = _flat_buffer(unit)
    layout = layout_metadata(unit.group_layout)
    state: dict[str, Any] = {
        "param_group_index": unit_index,
        "unit_index": unit_index,
        "module_fqn": module_fqn,
        "runtime_param_group_id": unit.runtime_param_group_id,
        "runtime_unit_id": unit.runtime_param_group_id,
        "planner_group_id": unit.runtime_param_group_id,
        "comm_buffer_id": unit.runtime_param_group_id,
        "rank": unit.rank,
        "world_size": unit.world_size,
        "replicate_world_size": unit.replicate_world_size,
        "dp_shard_mesh_dim": unit.dp_shard_mesh_dim,
        "dp_replicate_mesh_dim": unit.dp_replicate_mesh_dim,
        "device_mesh": unit.device_mesh_metadata,
        "mixed_precision": unit.mixed_precision_metadata(),
        "offload_policy": {"type": "OffloadPolicy", "cpu_offload": False},
        "total_numel": fb.plan.total_numel,
        "local_start": fb.local_start,
        "local_end": fb.local_end,
        "local_segments": [layout_segment_metadata(s) for s in fb.local_segments],
        "shard_sizes": tuple(fb.shard_sizes),
        "matrix_shard": matrix_shard_metadata(fb.placement),
        "param_shard_state": fb.param_state.as_metadata(),
        "layout": layout,
        "planner_layout": layout_metadata(unit.global_layout),
        "runtime_layout": layout,
        "planner_layout_contract": None,
        "runtime_layout_contract": None,
        "layout_flat_reordered": False,
        "runtime_layout_policy": "segment_program",
        "runtime_layout_mode": None,
        "runtime_layout_reason": None,
        "runtime_layout_requires_flat_reorder": False,
        "planner_metadata": None,
        "planner_summary": None,
        "planner_report": None,
        "planner_resource_estimate": None,
        "param_gather_strategy": "segment_program",
        "matrix_collective_backend": None,
        "grad_reduce_strategy": "segment_program",
        "param_fqns": tuple(mp.fqn for mp in unit.managed_params),
        "params": {mp.fqn: param_metadata(unit, fb, mp) for mp in unit.managed_params},
        "param_shard": _stored(fb.local_shard, clone=clone),
    }
    if include_grads:
        grad = fb.local_grad_shard
        state["grad_shard"] = None if grad is None else _stored(grad, clone=clone)
        state["grad_shard_state"] = None if grad is None else fb.grad_state.as_metadata()
    if full_state:
        # freshly assembled, so the views below own their memory already
        full = fb.gather_full_params()
        if clone and full.data_ptr() == fb.world_shards.data_ptr():  # rank-ordered layouts need no unpack: the shards themselves
            full = full.clone()
        state["full_params"] = {mp.fqn: full[mp.offset : mp.end].view(mp.shape).detach() for mp in unit.managed_params}
        if include_grads and fb.local_grad_shard is not None:
            full_grad = fb.gather_full_grads()
            state["full_grads"] = {mp.fqn: full_grad[mp.offset : mp.end].view(mp.shape).detach() for mp in unit.managed_params}
    return state


def matrix_state_dict(module_or_units, *, full_state: bool = False, include_grads: bool = False, clone: bool = True) -> dict[str, Any]:
    """Each unit's local shard and layout metadata; ``full_state`` adds the
    assembled full parameters under model-wide names (for debugging; the local
    shards stay, so the dict still loads)."""
    refs = collect_param_group_refs(module_or_units)
    units = [
        _unit_state_dict(unit, unit_index=i, module_fqn=fqn, include_grads=include_grads, full_state=full_state, clone=clone)
        for i, (fqn, unit) in enumerate(refs)
    ]
    state: dict[str, Any] = {
        "metadata": {
            "version": MATRIX_STATE_DICT_VERSION,
            "state_dict_type": "matrix_full" if full_state else "matrix_sharded",
            "num_param_groups": len(units),
            "num_units": len(units),
            "include_grads": include_grads,
        },
        "param_groups": units,
        "units": units,  # older readers look here; the same list object
    }
    if full_state:
        state["params"] = {param_key(u["module_fqn"], fqn, u["unit_index"]): t for u in units for fqn, t in u["full_params"].items()}
        if include_grads:
            state["grads"] = {param_key(u["module_fqn"], fqn, u["unit_index"]): t for u in units for fqn, t in u.get("full_grads", {}).items()}
    return state


def _check_field(unit_state: Mapping[str, Any], key: str, expected: Any) -> None:
    if key in unit_state and canonical(unit_state[key]) != canonical(expected):
        raise ValueError(
            f"State layout field {key!r}={unit_state[key]!r} does not match target {key!r}={expected!r}. "
            "Same-layout load requires identical MatrixFSDP layout metadata."
        )


_PARAM_FIELDS = ("shape", "dtype", "numel", "offset", "end", "owner_ranks", "local_segments", "shard_sizes", "matrix_shard", "shard_hint")


def _validate_same_layout(unit: MatrixFSDPParamGroup, unit_state: Mapping[str, Any], *, module_fqn: str) -> None:
    """Everything that decides which bytes a rank holds must match before a
    shard is copied in (state_dict.py:1113-1160, 1205-1240)."""
    fb = _flat_buffer(unit)
    if unit_state.get("module_fqn") not in {module_fqn, f"unit{unit_state.get('unit_index')}"}:
        raise ValueError(f"State unit module_fqn={unit_state.get('module_fqn')!r} does not match target {module_fqn!r}.")
    fqns = tuple(mp.fqn for mp in unit.managed_params)
    if tuple(unit_state.get("param_fqns", ())) != fqns:
        raise ValueError(f"State unit params {tuple(unit_state.get('param_fqns', ()))} do not match target params {fqns}.")
    if unit_state.get("rank") != unit.rank:
        raise ValueError(f"State rank {unit_state.get('rank')} does not match target rank {unit.rank}.")
    if unit_state.get("world_size") != unit.world_size:
        raise ValueError(f"State world_size {unit_state.get('world_size')} does not match target world_size {unit.world_size}.")
    _check_field(unit_state, "replicate_world_size", unit.replicate_world_size)
    _check_field(unit_state, "dp_shard_mesh_dim", unit.dp_shard_mesh_dim)
    _check_field(unit_state, "dp_replicate_mesh_dim", unit.dp_replicate_mesh_dim)
    if unit_state.get("device_mesh") is not None:
        raise ValueError(f"State device_mesh {unit_state['device_mesh']!r} does not match target device_mesh None.")
    if unit_state.get("total_numel") != fb.plan.total_numel:
        raise ValueError(f"State total_numel {unit_state.get('total_numel')} does not match target {fb.plan.total_numel}.")
    _check_field(unit_state, "local_start", fb.local_start)
    _check_field(unit_state, "local_end", fb.local_end)
    _check_field(unit_state, "local_segments", [layout_segment_metadata(s) for s in fb.local_segments])
    if tuple(unit_state.get("shard_sizes", ())) != tuple(fb.shard_sizes):
        raise ValueError(f"State shard_sizes {tuple(unit_state.get('shard_sizes', ()))} do not match target {tuple(fb.shard_sizes)}.")
    _check_field(unit_state, "matrix_shard", matrix_shard_metadata(fb.placement))
    layout = layout_metadata(unit.group_layout)
    _check_field(unit_state, "layout", layout)
    _check_field(unit_state, "runtime_layout", layout)
    _check_field(unit_state, "planner_layout", layout_metadata(unit.global_layout))
    saved_params = unit_state.get("params")
    if saved_params is None:
        return
    if tuple(saved_params) != fqns:
        raise ValueError(f"State param metadata keys {tuple(saved_params)} do not match target params {fqns}.")
    for mp in unit.managed_params:
        expected, saved = param_metadata(unit, fb, mp), saved_params[mp.fqn]
        for key in _PARAM_FIELDS:
            if key in saved and canonical(saved[key]) != canonical(expected[key]):
                raise ValueError(f"State param {mp.fqn!r} metadata field {key!r}={saved[key]!r} does not match target {expected[key]!r}.")


def _into_local_dtype(fb: MatrixFlatBuffer, tensor: torch.Tensor) -> torch.Tensor:
    """``tensor`` on the buffer's device in its local dtype (a host tensor is
    uploaded first)."""
    tensor = tensor.detach().reshape(-1)
    if tensor.device != fb.device:
        tensor = tensor.to(fb.device)
    if tensor.dtype == fb.local_shard.dtype:
        return tensor
    if (tensor.dtype, fb.local_shard.dtype) in CONVERTIBLE:
        return native.cast(tensor.contiguous(), fb.local_shard.dtype)
    return tensor.to(fb.local_shard.dtype)


def _load_unit_state_dict(unit: MatrixFSDPParamGroup, unit_state: Mapping[str, Any], *, module_fqn: str) -> None:
    fb = _flat_buffer(unit)
    _validate_same_layout(unit, unit_state, module_fqn=module_fqn)
    shard = unit_state.get("param_shard")
    if not torch.is_tensor(shard):
        raise TypeError("Unit state must contain tensor key 'param_shard'.")
    if shard.numel() != fb.local_numel:
        raise ValueError(f"Unit local shard has {shard.numel()} elements, expected {fb.local_numel}.")
    if shard.data_ptr() != fb.local_shard.data_ptr() and fb.local_numel:  # a DCP load has written into the shard itself
        native.copy_range(_into_local_dtype(fb, shard).contiguous(), fb.local_shard, 0)
    fb.use_local_shards()
    fb.clear_full_params()
    grad = unit_state.get("grad_shard")
    if torch.is_tensor(grad):
        if grad.numel() != fb.local_numel:
            raise ValueError(f"Unit local grad shard has {grad.numel()} elements, expected {fb.local_numel}.")
        fb.use_local_grad_shard(_into_local_dtype(fb, grad).clone())
    unit.reset_after_load()


def load_matrix_state_dict(module_or_units, state_dict: Mapping[str, Any]) -> None:
    """Same world size, same layout: every rank takes back the shard it saved."""
    version = state_dict.get("metadata", {}).get("version")
    if version != MATRIX_STATE_DICT_VERSION:
        raise ValueError(f"Unsupported MatrixFSDP state_dict version {version!r}; expected {MATRIX_STATE_DICT_VERSION}.")
    refs = collect_param_group_refs(module_or_units)
    unit_states = _unit_states(state_dict, context="state_dict")
    if len(refs) != len(unit_states):
        raise ValueError(f"State dict has {len(unit_states)} param groups, but target has {len(refs)} param groups.")
    for (module_fqn, unit), unit_state in zip(refs, unit_states):
        _load_unit_state_dict(unit, unit_state, module_fqn=module_fqn)


# ---------------------------------------------------------------------------
# DCP: save


def _single_process(process_group, no_dist: bool | None) -> None:
    if process_group is not None or no_dist is False:
        raise NotImplementedError(
            "This runtime is one process on one device: save and load with no_dist=True (or unset) and no process group; "
            "save_matrix_dcp_simulated_world writes the ranks of a simulated world together."
        )


def _dcp_payload(module_or_units, *, dcp_rank: int, full_state: bool, include_grads: bool, dedup_replicates: bool) -> tuple[dict[str, torch.Tensor], dict[str, Any]]:
    """Tensors by DCP key, and the metadata with every tensor replaced by its key."""
    state = matrix_state_dict(module_or_units, full_state=full_state, include_grads=include_grads, clone=False)
    tensors: dict[str, torch.Tensor] = {}
    units = []
    for unit_state in state["param_groups"]:
        index = unit_state["unit_index"]
        tag = dcp_io.payload_rank(unit_state, dcp_rank=dcp_rank, dedup_replicates=dedup_replicates)
        meta = dict(unit_state)
        shard_key = dcp_io.tensor_key(tag, index, "param_shard")
        tensors[shard_key] = meta.pop("param_shard")
        meta["dcp_payload_rank"] = tag
        meta["dcp_dedup_replicates"] = tag != f"rank_{dcp_rank}"
        meta["param_shard_key"] = shard_key
        meta["full_param_keys"] = {}
        for fqn, tensor in meta.pop("full_params", {}).items():
            key = dcp_io.tensor_key(tag, index, f"full_param.{fqn}")
            tensors[key] = tensor
            meta["full_param_keys"][fqn] = key
        grad = meta.pop("grad_shard", None)
        meta["grad_shard_key"] = None
        if torch.is_tensor(grad):
            meta["grad_shard_key"] = dcp_io.tensor_key(tag, index, "grad_shard")
            tensors[meta["grad_shard_key"]] = grad
        meta["full_grad_keys"] = {}
        for fqn, tensor in meta.pop("full_grads", {}).items():
            key = dcp_io.tensor_key(tag, index, f"full_grad.{fqn}")
            tensors[key] = tensor
            meta["full_grad_keys"][fqn] = key
        units.append(meta)
    metadata = {
        "metadata": {
            "version": MATRIX_STATE_DICT_VERSION,
            "dcp_format_version": MATRIX_DCP_FORMAT_VERSION,
            "state_dict_type": "matrix_dcp_sharded",
            "num_param_groups": len(units),
            "num_units": len(units),
            "full_state": full_state,
            "include_grads": include_grads,
            "dedup_replicates": dedup_replicates,
            "dcp_rank": dcp_rank,
        },
        "param_groups": units,
        "units": units,
    }
    return tensors, metadata


def _unwrap(optimizer):
    return getattr(optimizer, "optimizer", optimizer)


def optimizer_components(optimizer) -> tuple[tuple[str, Any], ...]:
    """``(("muon", ...), ("adamw", ...))`` for the mixed optimizer, else one
    component called ``"optimizer"`` (checkpoint/_optimizer_utils.py:13-18)."""
    inner = _unwrap(optimizer)
    named = getattr(inner, "iter_named_optimizers", None)
    return tuple(named()) if named is not None else (("optimizer", inner),)


def _full_fqn_by_param_id(refs: UnitRefs) -> dict[int, str]:
    return {id(mp.param): param_key(module_fqn, mp.fqn, i) for i, (module_fqn, unit) in enumerate(refs) for mp in unit.managed_params}


def _fqn_by_state_id(component, refs: UnitRefs) -> dict[int, str]:
    """The component's packed parameter ids -> model-wide parameter names."""
    by_param = _full_fqn_by_param_id(refs)
    packed = component.state_dict()["param_groups"]
    found = {}
    for group, packed_group in zip(component.param_groups, packed):
        for param, state_id in zip(group["params"], packed_group["params"]):
            if id(param) in by_param:
                found[state_id] = by_param[id(param)]
    return found


def _state_layout_metadata(optimizer, refs: UnitRefs) -> dict[str, dict[str, dict[str, Any]]]:
    """Placement metadata of the shard-shaped state tensors, by model-wide
    parameter name.  An optimizer that is not wrapped gets a manager for the
    occasion."""
    manager = getattr(optimizer, "state_manager", None)
    if not isinstance(manager, MatrixFSDPOptimizerStateManager):
        manager = MatrixFSDPOptimizerStateManager(_unwrap(optimizer), [unit for _, unit in refs])
    by_param = _full_fqn_by_param_id(refs)
    found: dict[str, dict[str, dict[str, Any]]] = {}
    for entry in manager.iter_local_state_tensors():
        found.setdefault(by_param[id(entry.param)], {})[entry.name] = entry.sharded_state.as_metadata()
    return found


def _dcp_optimizer_payload(optimizer, refs: UnitRefs, *, dcp_rank: int, dedup_replicates: bool) -> tuple[dict[str, torch.Tensor], dict[str, Any]]:
    layout_by_fqn = _state_layout_metadata(optimizer, refs)
    tag_by_fqn = {}
    for i, (module_fqn, unit) in enumerate(refs):
        tag = f"shard_{unit.rank}" if dedup_replicates and unit.replicate_world_size > 1 else f"rank_{dcp_rank}"
        for mp in unit.managed_params:
            tag_by_fqn[param_key(module_fqn, mp.fqn, i)] = tag
    tensors: dict[str, torch.Tensor] = {}
    components: dict[str, dict[str, Any]] = {}
    for name, component in optimizer_components(optimizer):
        packed = component.state_dict()
        fqn_by_id = _fqn_by_state_id(component, refs)
        states: dict[int, dict[str, Any]] = {}
        for state_id, state in packed["state"].items():
            fqn = fqn_by_id.get(state_id)
            if fqn is None:
                continue
            entries = {}
            for entry_name, value in state.items():
                if not torch.is_tensor(value):
                    entries[entry_name] = {"kind": "value", "value": deepcopy(value)}
                    continue
                key = dcp_io.tensor_key(tag_by_fqn.get(fqn, f"rank_{dcp_rank}"), 0, f"optimizer.{name}.{fqn}.{entry_name}")
                tensors[key] = value.detach()
                entries[entry_name] = {
                    "kind": "tensor",
                    "key": key,
                    "shape": tuple(value.shape),
                    "dtype": str(value.dtype),
                    "requires_grad": value.requires_grad,
                }
                placement = layout_by_fqn.get(fqn, {}).get(entry_name)
                if placement is not None:
                    entries[entry_name]["matrix_state"] = placement
            states[state_id] = {"fqn": fqn, "entries": entries}
        components[name] = {
            "class_name": type(component).__name__,
            "param_groups": deepcopy(packed["param_groups"]),
            "state": states,
        }
    inner = _unwrap(optimizer)
    summary = getattr(optimizer, "optimizer_group_summary", None) or getattr(inner, "optimizer_group_summary", None)
    metadata = {
        "optimizer_format_version": 2,
        "kind": "mixed_muon_adamw" if hasattr(inner, "iter_named_optimizers") else type(inner).__name__,
        "group_summary": deepcopy(summary()) if summary is not None else None,
        "components": components,
    }
    if tuple(components) == ("optimizer",):  # the shape older readers expect for a single optimizer
        metadata["param_groups"] = deepcopy(components["optimizer"]["param_groups"])
        metadata["state"] = components["optimizer"]["state"]
    return tensors, metadata


def _rank_payload(module_or_units, optimizer, *, dcp_rank: int, full_state: bool, include_grads: bool, dedup_replicates: bool):
    tensors, metadata = _dcp_payload(module_or_units, dcp_rank=dcp_rank, full_state=full_state, include_grads=include_grads, dedup_replicates=dedup_replicates)
    if optimizer is not None:
        refs = collect_param_group_refs(module_or_units)
        optimizer_tensors, metadata["optimizer"] = _dcp_optimizer_payload(optimizer, refs, dcp_rank=dcp_rank, dedup_replicates=dedup_replicates)
        tensors.update(optimizer_tensors)
    return tensors, metadata


def save_matrix_dcp(
    module_or_units,
    checkpoint_id: str | PathLike[str],
    *,
    optimizer: Any | None = None,
    full_state: bool = False,
    include_grads: bool = False,
    dedup_replicates: bool = True,
    process_group=None,
    no_dist: bool | None = None,
):
    """Local shards (and optimizer state) through DCP, layout metadata into
    ``matrix_metadata.pt``.  Written as DCP rank 0, as the reference does
    without a process group (state_dict.py:65-115)."""
    _single_process(process_group, no_dist)
    dcp = dcp_io.require_dcp()
    path = Path(checkpoint_id)
    path.mkdir(parents=True, exist_ok=True)
    tensors, metadata = _rank_payload(module_or_units, optimizer, dcp_rank=0, full_state=full_state, include_grads=include_grads, dedup_replicates=dedup_replicates)
    dcp_io.save_global_metadata(path, {0: metadata})
    return dcp.save(tensors, checkpoint_id=path, no_dist=True)


def save_matrix_dcp_simulated_world(
    rank_modules: Sequence,
    checkpoint_id: str | PathLike[str],
    *,
    optimizers: Sequence | None = None,
    include_grads: bool = False,
):
    """The checkpoint a job of ``len(rank_modules)`` processes would write:
    ``rank_modules[r]`` is the model as rank ``r`` of the simulated world holds
    it (``optimizers[r]`` its optimizer).  One DCP save carries every rank's
    tensors under that rank's keys and the metadata file lists all ranks."""
    dcp = dcp_io.require_dcp()
    path = Path(checkpoint_id)
    path.mkdir(parents=True, exist_ok=True)
    if optimizers is not None and len(optimizers) != len(rank_modules):
        raise ValueError(f"{len(optimizers)} optimizers for {len(rank_modules)} ranks.")
    tensors: dict[str, torch.Tensor] = {}
    metadata_by_rank = {}
    for rank, module in enumerate(rank_modules):
        for _, unit in collect_param_group_refs(module):
            if unit.rank != rank or unit.world_size != len(rank_modules):
                raise ValueError(f"rank_modules[{rank}] holds a unit of rank {unit.rank} in a world of {unit.world_size}.")
        rank_tensors, metadata_by_rank[rank] = _rank_payload(
            module, None if optimizers is None else optimizers[rank], dcp_rank=rank, full_state=False, include_grads=include_grads, dedup_replicates=True
        )
        tensors.update(rank_tensors)
    dcp_io.save_global_metadata(path, metadata_by_rank)
    return dcp.save(tensors, checkpoint_id=path, no_dist=True)


# ---------------------------------------------------------------------------
# DCP: same-layout load


def _check_dcp_header(header: Mapping[str, Any], *, dcp_rank: int) -> None:
    if header.get("version") != MATRIX_STATE_DICT_VERSION:
        raise ValueError(f"Unsupported MatrixFSDP state_dict version {header.get('version')!r}; expected {MATRIX_STATE_DICT_VERSION}.")
    if header.get("dcp_format_version") != MATRIX_DCP_FORMAT_VERSION:
        raise ValueError(f"Unsupported MatrixFSDP DCP format version {header.get('dcp_format_version')!r}; expected {MATRIX_DCP_FORMAT_VERSION}.")
    if header.get("dcp_rank") != dcp_rank:
        raise ValueError(f"Loaded metadata for DCP rank {header.get('dcp_rank')}, but current DCP rank is {dcp_rank}.")


def _state_tensor_device(component, state_id: int) -> torch.device:
    for group, packed_group in zip(component.param_groups, component.state_dict()["param_groups"]):
        for param, packed_id in zip(group["params"], packed_group["params"]):
            if packed_id == state_id:
                return param.device
    return torch.device("cpu")


def _empty_for_entry(entry: Mapping[str, Any], device: torch.device) -> torch.Tensor:
    shape = tuple(entry["shape"])
    # a 0-dim entry is a counter, not shard data: it stays on the host, where the optimizers read it
    return torch.empty(shape, dtype=dtype_from_string(entry["dtype"]), device=device if shape else "cpu")


def _current_param_groups(component, saved_groups: list[dict[str, Any]], *, same_sizes: bool) -> list[dict[str, Any]]:
    """The saved hyper-parameters over the component's current parameter ids.
    A same-layout load also wants every group to hold as many parameters as
    it did; another layout may leave a rank with fewer local parameters."""
    current = component.state_dict()["param_groups"]
    if len(current) != len(saved_groups):
        raise ValueError(f"Optimizer has {len(current)} param groups, checkpoint has {len(saved_groups)}.")
    groups = deepcopy(saved_groups)
    for now, saved in zip(current, groups):
        if same_sizes and len(now["params"]) != len(saved["params"]):
            raise ValueError(f"Optimizer param group has {len(now['params'])} params, checkpoint group has {len(saved['params'])}.")
        saved["params"] = list(now["params"])
    return groups


def _component_load_plan(component, refs: UnitRefs, saved: Mapping[str, Any], *, label: str) -> tuple[dict[str, torch.Tensor], dict[str, Any]]:
    groups = _current_param_groups(component, saved["param_groups"], same_sizes=True)
    id_by_fqn = {fqn: state_id for state_id, fqn in _fqn_by_state_id(component, refs).items()}
    tensors: dict[str, torch.Tensor] = {}
    states: dict[int, dict[str, Any]] = {}
    for state_metadata in saved["state"].values():
        fqn = state_metadata["fqn"]
        if fqn not in id_by_fqn:
            raise ValueError(f"{label} references unknown local parameter {fqn!r}.")
        state_id = id_by_fqn[fqn]
        entries = {}
        for name, entry in state_metadata["entries"].items():
            if entry["kind"] == "tensor":
                entries[name] = tensors[entry["key"]] = _empty_for_entry(entry, _state_tensor_device(component, state_id))
            else:
                entries[name] = deepcopy(entry["value"])
        states[state_id] = entries
    return tensors, {"state": states, "param_groups": groups}


def _optimizer_load_plan(optimizer, refs: UnitRefs, metadata: Mapping[str, Any]) -> tuple[dict[str, torch.Tensor], dict[str, dict[str, Any]]]:
    saved = metadata.get("optimizer")
    if saved is None:
        raise ValueError("MatrixFSDP DCP checkpoint does not contain optimizer state.")
    components = dict(optimizer_components(optimizer))
    if "components" not in saved:  # a checkpoint from before components were recorded
        tensors, state_dict = _component_load_plan(_unwrap(optimizer), refs, saved, label="Optimizer state")
        return tensors, {"optimizer": state_dict}
    saved_components = saved["components"]
    missing = sorted(set(components) - set(saved_components))
    if missing:
        raise ValueError(f"Optimizer checkpoint is missing component(s) {missing}; available components are {sorted(saved_components)}.")
    extra = sorted(set(saved_components) - set(components))
    if extra:
        raise ValueError(f"Optimizer checkpoint contains unknown component(s) {extra}; target components are {sorted(components)}.")
    tensors, plans = {}, {}
    for name, saved_component in saved_components.items():
        component_tensors, plans[name] = _component_load_plan(components[name], refs, saved_component, label=f"Optimizer component {name!r}")
        tensors.update(component_tensors)
    return tensors, plans


def _apply_optimizer_state(optimizer, state_dicts: Mapping[str, dict[str, Any]]) -> None:
    components = dict(optimizer_components(optimizer))
    for name, state_dict in state_dicts.items():
        components[name].load_state_dict(state_dict)
    refresh = getattr(optimizer, "refresh_state_dtensors", None)
    if refresh is not None:
        refresh()


def load_matrix_dcp(
    module_or_units,
    checkpoint_id: str | PathLike[str],
    *,
    optimizer: Any | None = None,
    allow_reshard: bool = False,
    process_group=None,
    no_dist: bool | None = None,
) -> None:
    """Loads what ``save_matrix_dcp`` wrote.  With the same world size and
    layout the shard is read straight into the local shard; with
    ``allow_reshard`` a checkpoint of any world size and layout over the same
    parameters is redistributed (see the module docstring)."""
    _single_process(process_group, no_dist)
    dcp = dcp_io.require_dcp()
    path = Path(checkpoint_id)
    refs = collect_param_group_refs(module_or_units)
    dcp_rank = 0
    try:
        metadata = dcp_io.load_metadata_for_rank(path, dcp_rank)
    except FileNotFoundError:
        if not allow_reshard:
            raise
        metadata = None
    if metadata is None or (allow_reshard and _needs_reshard(refs, metadata)):
        _load_resharded(refs, path, dcp=dcp, optimizer=optimizer)
        return
    _check_dcp_header(metadata.get("metadata", {}), dcp_rank=dcp_rank)
    unit_metadata = _unit_states(metadata, context="DCP metadata")
    if len(refs) != len(unit_metadata):
        raise ValueError(f"DCP metadata has {len(unit_metadata)} param groups, but target has {len(refs)} param groups.")
    tensors: dict[str, torch.Tensor] = {}
    unit_states = []
    for (module_fqn, unit), saved in zip(refs, unit_metadata):
        fb = _flat_buffer(unit)
        _validate_same_layout(unit, saved, module_fqn=module_fqn)  # before any tensor is touched
        unit_state = dict(saved)
        tensors[unit_state.pop("param_shard_key")] = unit_state["param_shard"] = fb.local_shard
        grad_key = unit_state.pop("grad_shard_key", None)
        if grad_key is not None:
            tensors[grad_key] = unit_state["grad_shard"] = fb.local_shard.new_empty(fb.local_numel)
        unit_states.append(unit_state)
    optimizer_states = None
    if optimizer is not None:
        optimizer_tensors, optimizer_states = _optimizer_load_plan(optimizer, refs, metadata)
        tensors.update(optimizer_tensors)
    dcp.load(tensors, checkpoint_id=path, no_dist=True)
    for (module_fqn, unit), unit_state in zip(refs, unit_states):
        _load_unit_state_dict(unit, unit_state, module_fqn=module_fqn)
    if optimizer_states is not None:
        _apply_optimizer_state(optimizer, optimizer_states)


def load_matrix_dcp_full_state(checkpoint_id: str | PathLike[str], *, source_rank: int = 0, process_group=None, no_dist: bool | None = None) -> dict[str, Any]:
    """The debug full parameters of ``save_matrix_dcp(full_state=True)`` as host
    tensors under model-wide names."""
    _single_process(process_group, no_dist)
    dcp = dcp_io.require_dcp()
    path = Path(checkpoint_id)
    metadata = dcp_io.load_metadata_for_rank(path, source_rank)
    tensors: dict[str, torch.Tensor] = {}
    found: dict[str, dict[str, torch.Tensor]] = {"params": {}, "grads": {}}
    for unit in _unit_states(metadata, context="DCP metadata"):
        for kind, keys in (("params", "full_param_keys"), ("grads", "full_grad_keys")):
            for fqn, key in unit.get(keys, {}).items():
                described = unit["params"][fqn]
                tensors[key] = torch.empty(tuple(described["shape"]), dtype=dtype_from_string(described["dtype"]))
                found[kind][param_key(unit["module_fqn"], fqn, unit["unit_index"])] = tensors[key]
    if not found["params"]:
        raise ValueError("This MatrixFSDP DCP checkpoint does not contain full_state tensors.")
    dcp.load(tensors, checkpoint_id=path, no_dist=True)
    result = {"metadata": metadata.get("metadata", {}), "params": found["params"]}
    if found["grads"]:
        result["grads"] = found["grads"]
    return result


# ---------------------------------------------------------------------------
# DCP: load into another layout


def _needs_reshard(refs: UnitRefs, metadata: Mapping[str, Any]) -> bool:
    saved_units = _unit_states(metadata, context="DCP metadata")
    if len(refs) != len(saved_units):
        return True
    for (_, unit), saved in zip(refs, saved_units):
        fb = _flat_buffer(unit)
        if saved.get("world_size") != unit.world_size or tuple(saved.get("shard_sizes", ())) != tuple(fb.shard_sizes):
            return True
        if tuple(saved.get("param_fqns", ())) != tuple(mp.fqn for mp in unit.managed_params):
            return True
        if canonical(saved.get("local_segments")) != canonical([layout_segment_metadata(s) for s in fb.local_segments]):
            return True  # same sizes, other elements: only a redistribution puts them right
    return False


def _source_plan(saved_unit: Mapping[str, Any]) -> ShardPlan:
    """The saved layout as a plan (every rank's metadata carries all ranks)."""
    layout = saved_unit.get("runtime_layout") or saved_unit.get("layout")
    if layout is None:
        raise ValueError("Source metadata carries no layout; it cannot be loaded into another layout.")
    segments = [
        tuple(LayoutSegment(int(s["global_start"]), int(s["global_end"]), int(s["local_start"])) for s in rank["segments"])
        for rank in sorted(layout["ranks"], key=lambda r: r["rank"])
    ]
    return ShardPlan.from_rank_segments(int(layout["total_numel"]), segments)


class _SourceUnit:
    """One unit as the source ranks saved it: the plan, where each rank's shard
    starts in the packed (rank-major) order, and the program that turns the
    packed order into flat-buffer order."""

    def __init__(self, saved_by_rank: list[Mapping[str, Any]], target: MatrixFSDPParamGroup) -> None:
        fb = _flat_buffer(target)
        fqns = tuple(mp.fqn for mp in target.managed_params)
        for saved in saved_by_rank:
            if tuple(saved.get("param_fqns", ())) != fqns:
                raise ValueError(f"Source params {tuple(saved.get('param_fqns', ()))} do not match target params {fqns}.")
            if saved.get("total_numel") != fb.plan.total_numel:
                raise ValueError(f"Source total_numel {saved.get('total_numel')} does not match target {fb.plan.total_numel}.")
        self.saved_by_rank = saved_by_rank
        self.plan = _source_plan(saved_by_rank[0])
        if len(self.plan.shard_sizes) != len(saved_by_rank):
            raise ValueError(f"Source layout has {len(self.plan.shard_sizes)} ranks, metadata for {len(saved_by_rank)}.")
        self.rank_base = [self.plan.rank_packed_offset(r) for r in range(len(saved_by_rank))]
        self.packed_numel = sum(self.plan.shard_sizes)
        self.target = fb
        self._unpack: dict[torch.dtype, Any] = {}

    def packed_buffer(self, dtype: torch.dtype, *, zero: bool) -> torch.Tensor:
        make = torch.zeros if zero else torch.empty
        return make(self.packed_numel, dtype=dtype, device=self.target.device)

    def rank_slot(self, packed: torch.Tensor, rank: int) -> torch.Tensor:
        return packed[self.rank_base[rank] : self.rank_base[rank] + self.plan.shard_sizes[rank]]

    def to_full(self, packed: torch.Tensor) -> torch.Tensor:
        """packed source shards -> flat-buffer order."""
        program = self._unpack.get(packed.dtype)
        if program is None:
            program = self._unpack[packed.dtype] = unpack_program(self.plan, packed.dtype, padded=False, device=self.target.device)
        full = torch.empty(self.plan.total_numel, dtype=packed.dtype, device=self.target.device)
        return program.run((packed,), full)

    def to_target_shard(self, packed: torch.Tensor) -> torch.Tensor:
        """packed source shards -> the target rank's shard."""
        out = torch.empty(self.target.local_numel, dtype=packed.dtype, device=self.target.device)
        return self.target.local_shard_from_full(self.to_full(packed), out=out)

    def param_slot(self, rank: int, local_fqn: str, numel: int) -> tuple[int, int] | None:
        """Where rank ``rank`` keeps its piece of ``local_fqn`` in the packed
        order, when that piece is one run of ``numel`` elements."""
        segments = self.saved_by_rank[rank]["params"][local_fqn].get("local_segments", ())
        if len(segments) != 1 or int(segments[0]["numel"]) != numel:
            return None
        start = self.rank_base[rank] + int(segments[0]["local_start"])
        return start, start + numel


def _reshard_optimizer_plan(component, refs: UnitRefs, sources: list[_SourceUnit], saved_by_rank: Mapping[int, Mapping[str, Any]]):
    """Allocates, for every unit and state name, one packed buffer that the
    source ranks' state tensors are read into at their shard positions.
    Returns ``(tensors by DCP key, finish)``; ``finish()`` builds the component's
    state dict once the tensors are loaded."""
    first = next(iter(saved_by_rank.values()))
    groups = _current_param_groups(component, first["param_groups"], same_sizes=False)
    id_by_fqn = {fqn: state_id for state_id, fqn in _fqn_by_state_id(component, refs).items()}
    unit_of_fqn = {param_key(module_fqn, mp.fqn, i): (i, mp) for i, (module_fqn, unit) in enumerate(refs) for mp in unit.managed_params}
    tensors: dict[str, torch.Tensor] = {}
    packed: dict[tuple[int, str, torch.dtype], torch.Tensor] = {}  # (unit, state name, dtype) -> packed source buffer
    wanted: dict[str, dict[str, torch.dtype]] = {}  # fqn -> shard-shaped state names
    loose: dict[str, dict[str, torch.Tensor]] = {}  # fqn -> states that are not shard data (counters, odd shapes); first rank wins
    values: dict[str, dict[str, Any]] = {}
    for rank in sorted(saved_by_rank):
        for state_metadata in saved_by_rank[rank]["state"].values():
            fqn = state_metadata["fqn"]
            if fqn not in unit_of_fqn:
                continue
            unit_index, mp = unit_of_fqn[fqn]
            source = sources[unit_index]
            for name, entry in state_metadata["entries"].items():
                if entry["kind"] != "tensor":
                    values.setdefault(fqn, {}).setdefault(name, deepcopy(entry["value"]))
                    continue
                shape, dtype = tuple(entry["shape"]), dtype_from_string(entry["dtype"])
                slot = source.param_slot(rank, mp.fqn, prod(shape)) if shape else None
                if slot is None:
                    tensor = torch.empty(shape, dtype=dtype, device=source.target.device if shape else "cpu")
                    tensors[entry["key"]] = tensor
                    loose.setdefault(fqn, {}).setdefault(name, tensor)
                    continue
                buffer = packed.get((unit_index, name, dtype))
                if buffer is None:
                    buffer = packed[(unit_index, name, dtype)] = source.packed_buffer(dtype, zero=True)
                tensors[entry["key"]] = buffer[slot[0] : slot[1]].view(shape)
                wanted.setdefault(fqn, {})[name] = dtype

    def finish() -> dict[str, Any]:
        local = {key: sources[key[0]].to_target_shard(buffer) for key, buffer in packed.items()}
        states: dict[int, dict[str, Any]] = {}
        for fqn, state_id in id_by_fqn.items():
            unit_index, mp = unit_of_fqn[fqn]
            views = [v for v in sources[unit_index].target.local_param_views if v.managed_param is mp]
            entries: dict[str, Any] = dict(values.get(fqn, {}))
            entries.update(loose.get(fqn, {}))
            if len(views) == 1:
                view = views[0]
                for name, dtype in wanted.get(fqn, {}).items():
                    piece = local[(unit_index, name, dtype)][view.shard_start : view.shard_end].clone()
                    entries[name] = piece.view(mp.shape) if view.numel == mp.numel else piece
            if entries:
                states[state_id] = entries
        return {"state": states, "param_groups": groups}

    return tensors, finish


def _load_resharded(refs: UnitRefs, path: Path, *, dcp, optimizer) -> None:
    metadata_by_rank = dcp_io.load_all_metadata(path)
    first_units = _unit_states(next(iter(metadata_by_rank.values())), context="DCP metadata")
    if not first_units:
        raise ValueError("MatrixFSDP DCP metadata does not contain any param groups.")
    source_world = int(first_units[0]["world_size"])
    if not set(range(source_world)) <= set(metadata_by_rank):
        raise ValueError(f"Expected DCP metadata sidecars for source ranks {list(range(source_world))}, found {sorted(metadata_by_rank)}.")
    units_by_rank = []
    for rank in range(source_world):
        units = _unit_states(metadata_by_rank[rank], context=f"source rank {rank} DCP metadata")
        if len(units) != len(refs):
            raise ValueError(f"Source rank {rank} has {len(units)} param groups, but target has {len(refs)} param groups.")
        units_by_rank.append(units)

    tensors: dict[str, torch.Tensor] = {}
    sources, param_packed, grad_packed = [], [], []
    for index, (_, unit) in enumerate(refs):
        fb = _flat_buffer(unit)
        source = _SourceUnit([units_by_rank[rank][index] for rank in range(source_world)], unit)
        sources.append(source)
        params = source.packed_buffer(fb.local_shard.dtype, zero=False)
        with_grads = all(saved.get("grad_shard_key") is not None for saved in source.saved_by_rank)
        grads = source.packed_buffer(fb.local_shard.dtype, zero=False) if with_grads else None
        for rank, saved in enumerate(source.saved_by_rank):
            tensors[saved["param_shard_key"]] = source.rank_slot(params, rank)
            if grads is not None:
                tensors[saved["grad_shard_key"]] = source.rank_slot(grads, rank)
            elif saved.get("grad_shard_key") is not None:  # some ranks only: read and dropped, as DCP wants every key it is given
                tensors[saved["grad_shard_key"]] = fb.local_shard.new_empty(source.plan.shard_sizes[rank])
        param_packed.append(params)
        grad_packed.append(grads)

    finishers = {}
    if optimizer is not None:
        # ranks may run different components (a rank that owns no matrix has no Muon): gather each component's
        # metadata from the ranks that have it
        saved_components: dict[str, dict[int, Mapping[str, Any]]] = {}
        for rank in range(source_world):
            saved = metadata_by_rank[rank].get("optimizer")
            if saved is None:
                continue
            for name, component_metadata in (saved["components"] if "components" in saved else {"optimizer": saved}).items():
                saved_components.setdefault(name, {})[rank] = component_metadata
        if not saved_components:
            raise ValueError("MatrixFSDP DCP checkpoint does not contain optimizer state.")
        for name, component in optimizer_components(optimizer):
            if name in saved_components:
                component_tensors, finishers[name] = _reshard_optimizer_plan(component, refs, sources, saved_components[name])
                tensors.update(component_tensors)

    dcp.load(tensors, checkpoint_id=path, no_dist=True)

    for (_, unit), source, params, grads in zip(refs, sources, param_packed, grad_packed):
        fb = _flat_buffer(unit)
        fb.load_full_params(source.to_full(params))
        fb.use_local_shards()
        fb.clear_full_params()
        if grads is not None:
            fb.use_local_grad_shard(source.to_target_shard(grads))
        unit.reset_after_load()
    if finishers:
        _apply_optimizer_state(optimizer, {name: finish() for name, finish in finishers.items()})
