"""``MatrixShard``: the placement a rank-contiguous flat shard plan reduces to.

A logical tensor is flattened over ``dims`` and cut into rank-ordered
contiguous chunks whose lengths are proportional to ``local_units``
(matrix_fsdp/core/placement.py:26-150).  Checkpoint metadata records the
placement of every local shard and of every shard-shaped optimizer state, so
the units are kept in lowest terms (shard sizes divided by their gcd,
placement.py:161-174) to make equal layouts compare equal.

This object is plain metadata; it is not a DTensor placement.
"""
from __future__ import annotations

from dataclasses import dataclass
from math import gcd

import torch

from .layout import MatrixGroupLayout, ShardPlan


@dataclass(frozen=True)
class MatrixShard:
    dims: tuple[int, ...]
    local_units: tuple[int, ...]

    def __post_init__(self) -> None:
        object.__setattr__(self, "dims", tuple(self.dims))
        object.__setattr__(self, "local_units", tuple(self.local_units))
        if not self.local_units:
            raise ValueError("local_units cannot be empty.")
        if any(unit < 0 for unit in self.local_units):
            raise ValueError(f"local_units must be non-negative, got {self.local_units}.")
        if sum(self.local_units) == 0:
            raise ValueError("local_units cannot all be zero.")
        if any(dim < 0 for dim in self.dims):
            raise ValueError(f"dims must be non-negative, got {self.dims}.")

    @property
    def world_size(self) -> int:
        return len(self.local_units)

    @property
    def total_units(self) -> int:
        return sum(self.local_units)

    def _elements_per_unit(self, total_numel: int) -> int:
        if total_numel < 0:
            raise ValueError(f"total_numel must be non-negative, got {total_numel}.")
        if total_numel % self.total_units:
            raise ValueError(f"total_numel={total_numel} must be divisible by sum(local_units)={self.total_units}.")
        return total_numel // self.total_units

    def _check_rank(self, rank: int) -> None:
        if not 0 <= rank < self.world_size:
            raise ValueError(f"rank={rank} is out of range for world_size={self.world_size}.")

    def shard_lengths(self, total_numel: int) -> tuple[int, ...]:
        per_unit = self._elements_per_unit(total_numel)
        return tuple(unit * per_unit for unit in self.local_units)

    def shard_offset(self, rank: int, total_numel: int) -> int:
        self._check_rank(rank)
        return sum(self.local_units[:rank]) * self._elements_per_unit(total_numel)

    def shard_range(self, rank: int, total_numel: int) -> tuple[int, int]:
        start = self.shard_offset(rank, total_numel)
        return start, start + self.shard_lengths(total_numel)[rank]

    def split_tensor(self, tensor: torch.Tensor, *, num_chunks: int | None = None) -> tuple[torch.Tensor, ...]:
        """Rank-ordered shards as views of the contiguous ``tensor``."""
        if not tensor.is_contiguous():
            raise ValueError("MatrixShard expects a contiguous tensor.")
        if num_chunks is not None and num_chunks != self.world_size:
            raise ValueError(f"num_chunks={num_chunks} must equal len(local_units)={self.world_size}.")
        flat = tensor.view(-1)
        return tuple(flat.split(list(self.shard_lengths(flat.numel()))))

    def local_shard(self, tensor: torch.Tensor, rank: int) -> torch.Tensor:
        self._check_rank(rank)
        return self.split_tensor(tensor)[rank]

    def reconstruct_tensor_from_flat(self, flat_tensor: torch.Tensor, shape: tuple[int, ...]) -> torch.Tensor:
        """A 1-D shard over the leading ``dims`` as ``[-1, *trailing shape]``."""
        if flat_tensor.ndim != 1:
            raise ValueError(f"flat_tensor must be 1D, got shape={tuple(flat_tensor.shape)}.")
        if self.dims != tuple(range(len(self.dims))):
            raise ValueError(f"dims must be a prefix tuple like (0, 1, ...), got {self.dims}.")
        trailing = tuple(shape[len(self.dims) :])
        per_row = 1
        for size in trailing:
            per_row *= size
        if flat_tensor.numel() % per_row:
            raise ValueError(f"flat_tensor.numel()={flat_tensor.numel()} must be divisible by trailing shape product={per_row}.")
        return flat_tensor.view(-1, *trailing)

    def is_matrix_shard(self) -> bool:
        return True

    def __repr__(self) -> str:
        return f"MatrixShard(dims={self.dims}, local_units={self.local_units})"


@dataclass(frozen=True)
class PlacementCompatibility:
    compatible: bool
    reason: str | None = None
    requires_flat_reorder: bool = False
    requires_multi_segment_runtime: bool = False


def shard_sizes_to_matrix_local_units(shard_sizes: tuple[int, ...]) -> tuple[int, ...]:
    """Shard sizes in lowest terms (placement.py:161-174)."""
    if not shard_sizes:
        raise ValueError("shard_sizes cannot be empty.")
    if any(size < 0 for size in shard_sizes):
        raise ValueError(f"shard_sizes must be non-negative, got {shard_sizes}.")
    if sum(shard_sizes) == 0:
        raise ValueError("Matrix local_units cannot represent an all-empty shard plan.")
    divisor = max(gcd(*shard_sizes), 1)
    return tuple(size // divisor for size in shard_sizes)


def explain_matrix_shard_compatibility(plan: ShardPlan | MatrixGroupLayout) -> PlacementCompatibility:
    """A plan (or group layout) is a ``MatrixShard`` when every non-empty rank
    holds exactly one segment and the segments tile the flat buffer in rank
    order (placement.py:177-222)."""
    if isinstance(plan, MatrixGroupLayout):
        plan = plan.to_shard_plan()
    if plan.total_numel <= 0:
        return PlacementCompatibility(False, "empty shard plans cannot be represented as matrix placements")
    cursor = 0
    for rank, segments in enumerate(plan.rank_segments):
        if plan.shard_sizes[rank] == 0:
            if segments:
                return PlacementCompatibility(False, f"rank {rank} has segments for an empty shard")
            continue
        if len(segments) != 1:
            return PlacementCompatibility(
                False,
                f"rank {rank} has {len(segments)} local segments, expected exactly one",
                requires_flat_reorder=True,
                requires_multi_segment_runtime=True,
            )
        (segment,) = segments
        if segment.local_start != 0:
            return PlacementCompatibility(False, f"rank {rank} segment local_start={segment.local_start}, expected 0")
        if segment.global_start != cursor:
            return PlacementCompatibility(
                False,
                f"rank {rank} segment starts at {segment.global_start}, expected rank-ordered cursor {cursor}",
                requires_flat_reorder=True,
            )
        if segment.numel != plan.shard_sizes[rank]:
            return PlacementCompatibility(False, f"rank {rank} segment size={segment.numel}, expected shard size={plan.shard_sizes[rank]}")
        cursor = segment.global_end
    if cursor != plan.total_numel:
        return PlacementCompatibility(False, f"rank segments cover {cursor} elements, expected {plan.total_numel}")
    return PlacementCompatibility(True)


def is_matrix_shard_compatible_plan(plan: ShardPlan | MatrixGroupLayout) -> bool:
    return explain_matrix_shard_compatibility(plan).compatible


def matrix_shard_from_plan(plan: ShardPlan | MatrixGroupLayout, *, dims: tuple[int, ...] = (0,)) -> MatrixShard:
    if isinstance(plan, MatrixGroupLayout):
        plan = plan.to_shard_plan()
    verdict = explain_matrix_shard_compatibility(plan)
    if not verdict.compatible:
        raise ValueError(
            "MatrixShard can directly represent only contiguous rank-ordered flat shard plans. "
            f"Reason: {verdict.reason}."
        )
    return MatrixShard(dims, shard_sizes_to_matrix_local_units(plan.shard_sizes))


def matrix_shard_from_layout(layout: MatrixGroupLayout, *, dims: tuple[int, ...] = (0,)) -> MatrixShard:
    return matrix_shard_from_plan(layout.to_shard_plan(), dims=dims)
