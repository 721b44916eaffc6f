"""Naming and metadata files of a MatrixFSDP checkpoint written through
PyTorch Distributed Checkpoint (DCP).

Tensor payloads are DCP entries keyed ``<payload rank>.unit_<i>.<name>``; the
layout metadata of all ranks lives in one ``matrix_metadata.pt`` beside them,
with per-rank ``matrix_metadata_rank_<r>.pt`` sidecars still read for older
checkpoints (matrix_fsdp/checkpoint/_dcp_utils.py:10-162).  This side never
runs more than one process, so there is no gather of the ranks' metadata:
callers hand in the dict of every rank they are writing.
"""
from __future__ import annotations

from collections.abc import Mapping
from pathlib import Path
from typing import Any

import torch

GLOBAL_METADATA_VERSION = 1
GLOBAL_METADATA_FILENAME = "matrix_metadata.pt"
GLOBAL_METADATA_FORMAT = "matrix_dcp_global_metadata"


def require_dcp():
    try:
        import torch.distributed.checkpoint as dcp
    except ImportError as error:
        raise RuntimeError("PyTorch Distributed Checkpoint is not available.") from error
    return dcp


def payload_rank(unit_state: Mapping[str, Any], *, dcp_rank: int, dedup_replicates: bool) -> str:
    """Replicas of one shard share a payload (``shard_<r>``); everything else is
    stored per DCP rank (``rank_<r>``)."""
    if dedup_replicates and int(unit_state.get("replicate_world_size", 1)) > 1:
        return f"shard_{int(unit_state['rank'])}"
    return f"rank_{dcp_rank}"


def tensor_key(rank_tag: str | int, unit_index: int, name: str) -> str:
    if isinstance(rank_tag, int):
        rank_tag = f"rank_{rank_tag}"
    return f"{rank_tag}.unit_{unit_index}.{name}"


def global_metadata_path(checkpoint_dir: Path) -> Path:
    return checkpoint_dir / GLOBAL_METADATA_FILENAME


def rank_metadata_path(checkpoint_dir: Path, dcp_rank: int) -> Path:
    return checkpoint_dir / f"matrix_metadata_rank_{dcp_rank}.pt"


def save_global_metadata(checkpoint_dir: Path, metadata_by_rank: Mapping[int, dict[str, Any]]) -> None:
    """One file for all ranks; sidecars of an older save in the same folder go."""
    for stale in checkpoint_dir.glob("matrix_metadata_rank_*.pt"):
        stale.unlink()
    torch.save(
        {
            "metadata": {
                "format": GLOBAL_METADATA_FORMAT,
                "version": GLOBAL_METADATA_VERSION,
                "num_ranks": len(metadata_by_rank),
                "ranks": tuple(sorted(metadata_by_rank)),
            },
            "ranks": dict(metadata_by_rank),
        },
        global_metadata_path(checkpoint_dir),
    )


def _read(path: Path) -> Any:
    # plain containers only: the restricted unpickler is enough and executes nothing from the file
    return torch.load(path, map_location="cpu", weights_only=True)


def load_global_metadata(checkpoint_dir: Path) -> dict[int, dict[str, Any]] | None:
    path = global_metadata_path(checkpoint_dir)
    if not path.exists():
        return None
    payload = _read(path)
    header = payload.get("metadata", {})
    if header.get("format") != GLOBAL_METADATA_FORMAT:
        raise ValueError(f"Unsupported MatrixFSDP global DCP metadata format {header.get('format')!r}.")
    if header.get("version") != GLOBAL_METADATA_VERSION:
        raise ValueError(
            f"Unsupported MatrixFSDP global DCP metadata version {header.get('version')!r}; "
            f"expected {GLOBAL_METADATA_VERSION}."
        )
    ranks = payload.get("ranks")
    if not isinstance(ranks, dict):
        raise TypeError("MatrixFSDP global DCP metadata must contain a dict at key 'ranks'.")
    return {int(rank): rank_metadata for rank, rank_metadata in ranks.items()}


def load_metadata_for_rank(checkpoint_dir: Path, dcp_rank: int) -> dict[str, Any]:
    by_rank = load_global_metadata(checkpoint_dir)
    if by_rank is not None:
        if dcp_rank not in by_rank:
            raise FileNotFoundError(f"MatrixFSDP global DCP metadata under {checkpoint_dir} does not contain rank {dcp_rank}.")
        return by_rank[dcp_rank]
    sidecar = rank_metadata_path(checkpoint_dir, dcp_rank)
    if not sidecar.exists():
        raise FileNotFoundError(
            f"Missing MatrixFSDP DCP metadata: expected {global_metadata_path(checkpoint_dir)} "
            f"or legacy sidecar {sidecar}."
        )
    return _read(sidecar)


def load_all_metadata(checkpoint_dir: Path) -> dict[int, dict[str, Any]]:
    by_rank = load_global_metadata(checkpoint_dir)
    if by_rank is not None:
        return by_rank
    by_rank = {int(path.stem.rsplit("_", 1)[-1]): _read(path) for path in sorted(checkpoint_dir.glob("matrix_metadata_rank_*.pt"))}
    if not by_rank:
        raise FileNotFoundError(f"No MatrixFSDP DCP metadata found under {checkpoint_dir}.")
    return by_rank
