"""``MatrixFSDPOptimizerStateManager``: placement metadata for the optimizer's
local tensor state.

The inner optimizers own ordinary tensors (views of the flat moment buffers
when ``flat_adamw_state`` is on).  For every state tensor that has as many
elements as its local parameter, the manager attaches the parameter's
``MatrixShard`` placement, so a checkpoint describes optimizer state in the
same terms as parameter and gradient shards
(matrix_fsdp/optim/state.py:47-184).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from ..core.managed_param import ManagedParam
from ..core.state import MatrixShardedState
from ..runtime.flat_buffer import MatrixFlatBuffer


@dataclass(frozen=True)
class LocalOptimizerStateTensor:
    fqn: str
    name: str
    tensor: torch.Tensor
    sharded_state: MatrixShardedState
    param: torch.Tensor | None = None  # the local parameter the state belongs to


@dataclass(frozen=True)
class OptimizerStateSummary:
    param_numel: int
    state_entries: int
    tensor_state_numel: int
    tensor_state_numel_by_name: dict[str, int]
    scalar_state_tensor_numel: int

    def as_dict(self) -> dict[str, Any]:
        return {
            "param_numel": self.param_numel,
            "state_entries": self.state_entries,
            "tensor_state_numel": self.tensor_state_numel,
            "tensor_state_numel_by_name": dict(self.tensor_state_numel_by_name),
            "scalar_state_tensor_numel": self.scalar_state_tensor_numel,
        }


class MatrixFSDPOptimizerStateManager:
    def __init__(self, optimizer, param_groups: list) -> None:
        self.optimizer = optimizer
        self.fsdp_param_groups = list(param_groups)
        self._state_objects: dict[str, dict[str, MatrixShardedState]] = {}

    @property
    def runtime_param_groups(self) -> list:
        return self.fsdp_param_groups

    @property
    def state_objects(self) -> dict[str, dict[str, MatrixShardedState]]:
        return self._state_objects

    @property
    def state_dtensors(self) -> dict[str, dict[str, Any]]:
        return {}

    # ------------------------------------------------------------------ summaries
    def summarize(self) -> OptimizerStateSummary:
        by_name: dict[str, int] = {}
        scalars = 0
        for state in self.optimizer.state.values():
            for name, value in state.items():
                if not torch.is_tensor(value):
                    continue
                if value.ndim == 0:
                    scalars += value.numel()
                else:
                    by_name[name] = by_name.get(name, 0) + value.numel()
        return OptimizerStateSummary(
            param_numel=sum(p.numel() for group in self.optimizer.param_groups for p in group["params"]),
            state_entries=len(self.optimizer.state),
            tensor_state_numel=sum(by_name.values()),
            tensor_state_numel_by_name=by_name,
            scalar_state_tensor_numel=scalars,
        )

    def local_state_summary(self) -> dict[str, Any]:
        return self.summarize().as_dict()

    # ------------------------------------------------------------------ placement metadata
    def _local_param_owners(self) -> dict[int, tuple[MatrixFlatBuffer, ManagedParam]]:
        owners = {}
        for unit in self.fsdp_param_groups:
            if unit.flat_buffer is None:
                continue
            for view in unit.flat_buffer.local_param_views:
                owners[id(view.managed_param.param)] = (unit.flat_buffer, view.managed_param)
        return owners

    def iter_local_state_tensors(self) -> tuple[LocalOptimizerStateTensor, ...]:
        owners = self._local_param_owners()
        found = []
        for param, state in self.optimizer.state.items():
            if not torch.is_tensor(param) or param.numel() == 0 or id(param) not in owners:
                continue
            flat_buffer, managed_param = owners[id(param)]
            for name, value in state.items():
                if not torch.is_tensor(value) or value.ndim == 0 or value.numel() != param.numel():
                    continue
                sharded = flat_buffer.make_param_state(managed_param, name, value)
                if sharded is not None:
                    found.append(LocalOptimizerStateTensor(managed_param.fqn, name, value, sharded, param))
        return tuple(found)

    def local_state_objects(self) -> dict[str, dict[str, MatrixShardedState]]:
        objects: dict[str, dict[str, MatrixShardedState]] = {}
        for entry in self.iter_local_state_tensors():
            objects.setdefault(entry.fqn, {})[entry.name] = entry.sharded_state
        return objects

    def local_state_dtensors(self) -> dict[str, dict[str, Any]]:
        return {}

    def local_state_metadata(self) -> dict[str, dict[str, dict[str, Any]]]:
        return {fqn: {name: state.as_metadata() for name, state in states.items()} for fqn, states in self.local_state_objects().items()}

    def refresh_state_dtensors(self) -> dict[str, dict[str, Any]]:
        """Rebuilds the cached state objects; DTensor wrappers are never made."""
        self._state_objects = self.local_state_objects()
        return {}

    def validate_local_state_shapes(self) -> None:
        for param, state in self.optimizer.state.items():
            if not torch.is_tensor(param):
                continue
            for name, value in state.items():
                if torch.is_tensor(value) and value.ndim != 0 and value.numel() != param.numel():
                    raise RuntimeError(
                        f"Optimizer state {name!r} has {value.numel()} elements for a "
                        f"local parameter with {param.numel()} elements."
                    )
