"""``MatrixShardedState``: a local tensor together with the placement that
says where it sits in its logical global tensor.

The runtime keeps ordinary local tensors; this object only carries what a
checkpoint has to record about one of them -- parameter shard, gradient shard
or a shard-shaped optimizer state -- in the vocabulary of the layouts
(matrix_fsdp/core/state.py:16-118).  No DTensor is ever built, and on a single
device there is no device mesh, so both entries of the metadata are ``None``.
"""
from __future__ import annotations

from collections.abc import Sequence
from typing import Any

import torch

from .placement import MatrixShard


def matrix_shard_metadata(placement: MatrixShard | None) -> dict[str, Any] | None:
    """core/state.py:121-128 (the form with a ``type`` tag)."""
    if placement is None:
        return None
    return {"type": "MatrixShard", "dims": tuple(placement.dims), "local_units": tuple(placement.local_units)}


class MatrixShardedState:
    def __init__(
        self,
        name: str,
        local_tensor: torch.Tensor,
        *,
        mesh: None = None,
        placement: MatrixShard | None,
        global_shape: Sequence[int],
        global_stride: Sequence[int] | None = None,
        shard_mesh_dim: int | str = 0,
        requires_grad: bool | None = None,
    ) -> None:
        if mesh is not None:
            raise NotImplementedError("A single device has no device mesh; pass mesh=None.")
        self.name = name
        self.placement = placement
        self.global_shape = torch.Size(tuple(global_shape))
        self.global_stride = None if global_stride is None else tuple(global_stride)
        self.shard_mesh_dim = shard_mesh_dim
        self.requires_grad = local_tensor.requires_grad if requires_grad is None else requires_grad
        self.mesh = None
        self.mesh_metadata = None
        self._local_tensor = local_tensor

    @property
    def local_tensor(self) -> torch.Tensor:
        return self._local_tensor

    @property
    def fallback_tensor(self) -> torch.Tensor:
        return self._local_tensor

    @property
    def dtensor(self) -> None:
        return None

    @property
    def uses_dtensor(self) -> bool:
        return False

    def refresh(self, local_tensor: torch.Tensor) -> "MatrixShardedState":
        """The same placement over another local tensor."""
        return MatrixShardedState(
            self.name,
            local_tensor,
            placement=self.placement,
            global_shape=self.global_shape,
            global_stride=self.global_stride,
            shard_mesh_dim=self.shard_mesh_dim,
            requires_grad=local_tensor.requires_grad,
        )

    def shares_storage_with(self, tensor: torch.Tensor) -> bool:
        return self._local_tensor.untyped_storage().data_ptr() == tensor.untyped_storage().data_ptr()

    def has_same_data_ptr(self, tensor: torch.Tensor) -> bool:
        return self._local_tensor.data_ptr() == tensor.data_ptr()

    def as_metadata(self) -> dict[str, Any]:
        """Key for key what core/state.py:100-118 writes."""
        t = self._local_tensor
        return {
            "name": self.name,
            "uses_dtensor": False,
            "global_shape": tuple(self.global_shape),
            "global_stride": self.global_stride,
            "local_shape": tuple(t.shape),
            "local_numel": t.numel(),
            "dtype": str(t.dtype),
            "device": str(t.device),
            "requires_grad": self.requires_grad,
            "shard_mesh_dim": self.shard_mesh_dim,
            "device_mesh": self.mesh_metadata,
            "matrix_shard": matrix_shard_metadata(self.placement),
            "dtensor_spec": None,
        }


def matrix_sharded_state_metadata(state: MatrixShardedState) -> dict[str, Any]:
    return state.as_metadata()
