"""Placement, group-layout and sharded-state metadata (CPU), on the values the reference's own tests expect
(test/fsdp/test_placement.py:27-104, test_layout.py:31-94, test_sharded_state.py:83-100), plus the metadata files of
a DCP checkpoint folder."""
import pytest
import torch

from matrix_fsdp_amd.checkpoint import dcp_io
from matrix_fsdp_amd.checkpoint.metadata import canonical, dtype_from_string, layout_metadata, param_key
from matrix_fsdp_amd.core.layout import LayoutSegment, MatrixGroupLayout, ParamLayout, ParamSegment, ShardPlan
from matrix_fsdp_amd.core.placement import (
    MatrixShard,
    explain_matrix_shard_compatibility,
    is_matrix_shard_compatible_plan,
    matrix_shard_from_plan,
    shard_sizes_to_matrix_local_units,
)
from matrix_fsdp_amd.core.state import MatrixShardedState

from tests.conftest import P


def test_matrix_shard_splits_by_local_units():
    placement = MatrixShard(dims=(0,), local_units=(1, 2, 1))
    tensor = torch.arange(16)
    assert [s.tolist() for s in placement.split_tensor(tensor)] == [[0, 1, 2, 3], list(range(4, 12)), [12, 13, 14, 15]]
    assert placement.shard_range(1, 16) == (4, 12)
    assert torch.equal(placement.local_shard(tensor, 1), tensor[4:12])
    assert placement.split_tensor(tensor)[1].data_ptr() == tensor[4:].data_ptr()  # views, not copies
    assert tuple(MatrixShard((0,), (1, 1)).reconstruct_tensor_from_flat(torch.arange(12), (6, 2)).shape) == (6, 2)
    with pytest.raises(ValueError, match="divisible"):
        MatrixShard((0,), (1, 2)).split_tensor(torch.arange(5))
    for bad in ((), (0, 0), (1, -1)):
        with pytest.raises(ValueError):
            MatrixShard((0,), bad)


def test_local_units_are_shard_sizes_in_lowest_terms():
    assert shard_sizes_to_matrix_local_units((4, 8, 4)) == (1, 2, 1)
    assert shard_sizes_to_matrix_local_units((0, 6, 3)) == (0, 2, 1)
    assert shard_sizes_to_matrix_local_units((3, 5)) == (3, 5)
    assert shard_sizes_to_matrix_local_units((42,)) == (1,)


def test_matrix_shard_from_plans():
    placement = matrix_shard_from_plan(ShardPlan(16, (4, 8, 4), (0, 4, 12)))
    assert placement.dims == (0,) and placement.local_units == (1, 2, 1)
    layout = MatrixGroupLayout.from_rank_segments(12, ((LayoutSegment(0, 3, 0),), (LayoutSegment(3, 12, 0),)))
    assert matrix_shard_from_plan(layout.to_shard_plan()).local_units == (1, 3)
    split = ShardPlan(8, (4, 4), (0, 4), ((LayoutSegment(0, 2, 0), LayoutSegment(6, 8, 2)), (LayoutSegment(2, 6, 0),)))
    verdict = explain_matrix_shard_compatibility(split)
    assert not is_matrix_shard_compatible_plan(split) and not verdict.compatible
    assert verdict.requires_flat_reorder and verdict.requires_multi_segment_runtime
    with pytest.raises(ValueError, match="contiguous rank-ordered"):
        matrix_shard_from_plan(split)
    swapped = ShardPlan(8, (4, 4), (0, 4), ((LayoutSegment(4, 8, 0),), (LayoutSegment(0, 4, 0),)))
    verdict = explain_matrix_shard_compatibility(swapped)
    assert not verdict.compatible and verdict.requires_flat_reorder and not verdict.requires_multi_segment_runtime


def test_group_layout_queries():
    layout = MatrixGroupLayout.from_rank_segments(
        8,
        ((LayoutSegment(0, 2, 0), LayoutSegment(6, 8, 2)), (LayoutSegment(2, 6, 0),)),
        params=(
            ParamLayout("weight", 0, 8, (ParamSegment("weight", 0, 0, 2, 0), ParamSegment("weight", 0, 6, 8, 2), ParamSegment("weight", 1, 2, 6, 0))),
        ),
    )
    assert layout.world_size == 2 and layout.shard_sizes == (4, 4) and layout.params[0].numel == 8
    assert layout.param("weight") is layout.params[0]
    assert layout.owner_ranks("weight") == (0, 1) and layout.params_for_rank(0) == ("weight",)
    assert layout.rank_segments_for_param(0, "weight") == (ParamSegment("weight", 0, 0, 2, 0), ParamSegment("weight", 0, 6, 8, 2))
    with pytest.raises(KeyError):
        layout.param("missing")
    plan = layout.to_shard_plan()
    assert plan.shard_sizes == (4, 4) and plan.shard_offsets == (0, 4)
    assert plan.local_segments(0) == (LayoutSegment(0, 2, 0), LayoutSegment(6, 8, 2))


def test_group_layout_cuts_params_along_the_plan():
    layout = MatrixGroupLayout.from_shard_plan(ShardPlan(8, (3, 5), (0, 3)), params=(P("p0", 0, 4), P("p1", 4, 4)))
    assert layout.owner_ranks("p0") == (0, 1) and layout.owner_ranks("p1") == (1,)
    assert layout.rank_segments_for_param(0, "p0") == (ParamSegment("p0", 0, 0, 3, 0),)
    assert layout.rank_segments_for_param(1, "p0") == (ParamSegment("p0", 1, 3, 4, 0),)
    assert layout.rank_segments_for_param(1, "p1") == (ParamSegment("p1", 1, 4, 8, 1),)
    assert layout.params_for_rank(1) == ("p0", "p1")
    described = layout_metadata(layout)
    assert described["total_numel"] == 8 and described["world_size"] == 2 and described["shard_sizes"] == (3, 5)
    assert described["ranks"][1] == {"rank": 1, "local_units": 5, "segments": [{"global_start": 3, "global_end": 8, "local_start": 0, "local_end": 5, "numel": 5}]}
    assert described["params"][0]["segments"][1] == {"fqn": "p0", "rank": 1, "global_start": 3, "global_end": 4, "local_start": 0, "local_end": 1, "numel": 1}
    assert canonical(described) == canonical(layout_metadata(MatrixGroupLayout.from_shard_plan(ShardPlan(8, (3, 5), (0, 3)), params=(P("p0", 0, 4), P("p1", 4, 4)))))


def test_sharded_state_metadata():
    local = torch.arange(4, dtype=torch.float32)
    state = MatrixShardedState("param", local, mesh=None, placement=MatrixShard((0,), (1,)), global_shape=(4,))
    assert not state.uses_dtensor and state.dtensor is None and state.mesh_metadata is None
    assert state.fallback_tensor is local and state.has_same_data_ptr(local) and state.shares_storage_with(local[2:])
    assert not state.has_same_data_ptr(local[2:])
    described = state.as_metadata()
    assert described == {
        "name": "param",
        "uses_dtensor": False,
        "global_shape": (4,),
        "global_stride": None,
        "local_shape": (4,),
        "local_numel": 4,
        "dtype": "torch.float32",
        "device": "cpu",
        "requires_grad": False,
        "shard_mesh_dim": 0,
        "device_mesh": None,
        "matrix_shard": {"type": "MatrixShard", "dims": (0,), "local_units": (1,)},
        "dtensor_spec": None,
    }
    other = state.refresh(torch.zeros(4, requires_grad=True))
    assert other.requires_grad and other.placement == state.placement and other.name == "param"
    with pytest.raises(NotImplementedError):
        MatrixShardedState("param", local, mesh=object(), placement=None, global_shape=(4,))


def test_names_and_dtypes():
    assert param_key("", "0.weight", 0) == "0.weight"
    assert param_key("layers.1", "weight", 3) == "layers.1.weight"
    assert param_key("", "", 3) == "unit3"
    assert dtype_from_string("torch.bfloat16") is torch.bfloat16
    for bad in ("bfloat16", "torch.nn", "torch.nope"):
        with pytest.raises(ValueError):
            dtype_from_string(bad)
    assert dcp_io.tensor_key(2, 1, "param_shard") == "rank_2.unit_1.param_shard"
    assert dcp_io.tensor_key("shard_0", 0, "grad_shard") == "shard_0.unit_0.grad_shard"
    assert dcp_io.payload_rank({"replicate_world_size": 1, "rank": 3}, dcp_rank=5, dedup_replicates=True) == "rank_5"
    assert dcp_io.payload_rank({"replicate_world_size": 2, "rank": 3}, dcp_rank=5, dedup_replicates=True) == "shard_3"
    assert dcp_io.payload_rank({"replicate_world_size": 2, "rank": 3}, dcp_rank=5, dedup_replicates=False) == "rank_5"


def test_metadata_files(tmp_path):
    ranks = {0: {"metadata": {"dcp_rank": 0}, "param_groups": [{"shard_sizes": (3, 5)}]}, 1: {"metadata": {"dcp_rank": 1}, "param_groups": []}}
    torch.save({"stale": True}, tmp_path / "matrix_metadata_rank_0.pt")
    dcp_io.save_global_metadata(tmp_path, ranks)
    assert not list(tmp_path.glob("matrix_metadata_rank_*.pt"))  # one file for all ranks replaces older sidecars
    payload = torch.load(tmp_path / "matrix_metadata.pt", map_location="cpu", weights_only=True)
    assert payload["metadata"] == {"format": "matrix_dcp_global_metadata", "version": 1, "num_ranks": 2, "ranks": (0, 1)}
    assert dcp_io.load_metadata_for_rank(tmp_path, 1) == ranks[1]
    assert dcp_io.load_all_metadata(tmp_path) == ranks
    with pytest.raises(FileNotFoundError, match="does not contain rank 2"):
        dcp_io.load_metadata_for_rank(tmp_path, 2)

    # per-rank sidecars of older checkpoints are still read
    (tmp_path / "matrix_metadata.pt").unlink()
    with pytest.raises(FileNotFoundError, match="Missing MatrixFSDP DCP metadata"):
        dcp_io.load_metadata_for_rank(tmp_path, 0)
    with pytest.raises(FileNotFoundError, match="No MatrixFSDP DCP metadata"):
        dcp_io.load_all_metadata(tmp_path)
    for rank, rank_metadata in ranks.items():
        torch.save(rank_metadata, tmp_path / f"matrix_metadata_rank_{rank}.pt")
    assert dcp_io.load_metadata_for_rank(tmp_path, 1) == ranks[1]
    assert dcp_io.load_all_metadata(tmp_path) == ranks

    torch.save({"metadata": {"format": "something else", "version": 1}, "ranks": {}}, tmp_path / "matrix_metadata.pt")
    with pytest.raises(ValueError, match="format"):
        dcp_io.load_global_metadata(tmp_path)
    torch.save({"metadata": {"format": "matrix_dcp_global_metadata", "version": 2}, "ranks": {}}, tmp_path / "matrix_metadata.pt")
    with pytest.raises(ValueError, match="version"):
        dcp_io.load_global_metadata(tmp_path)
