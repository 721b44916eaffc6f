"""CPU tests of the host-side mirror: shard metadata, layout classification, closed-form plans, the
C-ABI library's symbols, and the run compiler (host part of the library)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from matrix_fsdp_amd import LayoutSegment, ShardPlan, _lib, managed_params_from_named, validate_shard_plan
from matrix_fsdp_amd.core.plans import (
    block_grid_plan,
    contiguous_even_plan,
    fsdp2_chunk_plan,
    rank_major_owner_order,
    whole_param_owner_plan,
)
from matrix_fsdp_amd.kernels.segment_fusion import coalesce_contiguous_segments, coalesce_rank_segments
from matrix_fsdp_amd.kernels.segment_program import fill_runs_for_gaps, grad_fill_runs, make_runs, merge_runs
from matrix_fsdp_amd.runtime.grad_bucket import BucketParamGrad, MatrixGradBucket, classify_copy_in_layout, fill_reduce_scatter_input
from matrix_fsdp_amd.runtime.param_buffer_layout import ParamBufferLayout, rank_chunk_shard_sizes
from matrix_fsdp_amd.workloads import HIDDEN2048_W4, HIDDEN4096_W4_BLOCK, MLP_W2, param_specs
from oracle import copy_oracle as O
from tests.conftest import segs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def managed(pairs):
    return managed_params_from_named([(n, torch.nn.Parameter(torch.zeros(k))) for n, k in pairs])


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mfsdp_hip.h")).read()
    declared = set(re.findall(r"\b(mfsdp_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    handle = _lib.lib()
    for name in declared:
        assert getattr(handle, name) is not None
    assert handle.mfsdp_abi_version() == _lib.ABI_VERSION
    assert ctypes.sizeof(_lib.CopyRun) == 56


def test_layout_segment_and_plan_defaults():
    seg = LayoutSegment(3, 8, 2)
    assert seg.numel == 5 and seg.local_end == 7 and seg.intersects(7, 9) and not seg.intersects(8, 9)
    plan = ShardPlan(10, (4, 6), (0, 4))
    assert plan.rank_segments == ((LayoutSegment(0, 4, 0),), (LayoutSegment(4, 10, 0),))
    assert plan.local_range(1) == (4, 10) and plan.rank_packed_offset(1) == 4
    validate_shard_plan(plan)
    with pytest.raises(ValueError):
        validate_shard_plan(ShardPlan(10, (4, 5), (0, 4)))
    with pytest.raises(ValueError):
        validate_shard_plan(ShardPlan.from_rank_segments(6, ((LayoutSegment(0, 4, 0),), (LayoutSegment(3, 6, 0),))))
    with pytest.raises(ValueError):
        validate_shard_plan(ShardPlan(4, (4,), (0,), ((LayoutSegment(0, 4, 1),),)))


def test_managed_params_offsets_and_duplicates():
    mps = managed([("w", 6), ("b", 4)])
    assert [(m.fqn, m.offset, m.end, m.numel) for m in mps] == [("w", 0, 6, 6), ("b", 6, 10, 4)]
    assert mps[0].shard_hint.optimizer_type is None and mps[1].local_name == "b"
    with pytest.raises(ValueError, match="Duplicate"):
        managed([("w", 1), ("w", 2)])
    lin = torch.nn.Linear(3, 2)
    tied = torch.nn.ModuleList([lin, lin])
    from matrix_fsdp_amd import managed_params_from_module

    assert [m.fqn for m in managed_params_from_module(lin)] == ["weight", "bias"]
    with pytest.raises(NotImplementedError, match="shared"):
        managed_params_from_module(tied)


def test_coalesce_reference_vector(golden):
    g = golden["coalesce_contiguous_segments"]
    have = coalesce_contiguous_segments(tuple(LayoutSegment(*t) for t in g["segments"]))
    assert have == tuple(LayoutSegment(*t) for t in g["fused"])
    assert coalesce_contiguous_segments(()) == ()
    assert coalesce_rank_segments(((LayoutSegment(0, 1, 0), LayoutSegment(1, 2, 1)), ())) == ((LayoutSegment(0, 2, 0),), ())


def test_rank_chunk_detection_reference_vectors(golden):
    for case in golden["rank_chunk_shard_sizes"]["cases"]:
        want = None if case["shard_sizes"] is None else tuple(case["shard_sizes"])
        assert rank_chunk_shard_sizes(segs(case["rank_segments"])) == want


def test_param_buffer_layout_reference_vectors(golden):
    g = golden["param_buffer_layout"]
    layout = ParamBufferLayout(g["total_numel"], tuple(g["shard_sizes"]), segs(g["rank_segments"]))
    assert layout.padded_numel == g["padded_numel"] and layout.padding_waste_numel == g["padding_waste_numel"]
    assert layout.padding_waste_ratio == pytest.approx(g["padding_waste_ratio"])
    assert layout.owner_imbalance_ratio == pytest.approx(g["owner_imbalance_ratio"])
    assert layout.segment_count == g["segment_count"] and layout.max_segments_per_rank == g["max_segments_per_rank"]
    assert layout.rank_chunk_fast_path and layout.packed_rank_shards_are_full_tensor_order
    assert layout.rank_chunk_workspace_numel(compact=True) == 10 and layout.rank_chunk_workspace_numel(compact=False) == 12
    g = golden["param_buffer_layout_not_chunks"]
    layout = ParamBufferLayout(g["total_numel"], tuple(g["shard_sizes"]), segs(g["rank_segments"]))
    assert not layout.rank_chunk_fast_path and not layout.packed_rank_shards_are_full_tensor_order


def test_communication_plan_reference_expectations():
    """test/fsdp/test_elastic_param_buffer.py:32-82: the plan keeps the layout's segments, merges neighbours, lists
    one chunk per segment and knows the rank-chunk sizes exactly when every rank holds one stretch in rank order."""
    from matrix_fsdp_amd.core.layout import LayoutSegment as S
    from matrix_fsdp_amd.runtime.param_buffer_layout import ElasticCommunicationPlan, ElasticParamBufferLayout, StaticParamBufferLayout

    assert StaticParamBufferLayout is ParamBufferLayout and ElasticParamBufferLayout is ParamBufferLayout
    rank_segments = ((S(0, 4, 0),), (S(4, 10, 0),), ())
    plan = ElasticParamBufferLayout(10, (4, 6, 0), rank_segments).build_communication_plan()
    assert isinstance(plan, ElasticCommunicationPlan) and plan.rank_segments is rank_segments
    assert plan.rank_chunk_shard_sizes == (4, 6, 0) and plan.rank_chunk_segments == rank_segments
    assert plan.rank_chunk_fast_path and plan.packed_full_order
    assert plan.rank_chunk_count == 2 and plan.nonempty_rank_chunk_count == 2 and plan.world_size == 3
    assert plan.as_summary()["communication_plan_rank_chunk_fast_path"] is True
    assert [c.as_segment() for c in plan.rank_chunks] == [S(0, 4, 0), S(4, 10, 0)] and [c.rank for c in plan.rank_chunks] == [0, 1]

    plan = ElasticParamBufferLayout(6, (4, 2), ((S(0, 2, 0), S(2, 4, 2)), (S(4, 6, 0),))).build_communication_plan()
    assert plan.coalesced_rank_segments == ((S(0, 4, 0),), (S(4, 6, 0),))
    assert plan.rank_chunk_shard_sizes is None and not plan.rank_chunk_fast_path
    assert plan.segment_count == 3 and plan.coalesced_segment_count == 2
    assert plan.max_segments_per_rank == 2 and plan.max_coalesced_segments_per_rank == 1

    # no segment table: the shard sizes alone describe rank-ordered stretches
    plan = ParamBufferLayout(10, (6, 0, 4), None).build_communication_plan()
    assert plan.rank_segments == ((S(0, 6, 0),), (), (S(6, 10, 0),)) and plan.rank_chunk_shard_sizes == (6, 0, 4)


@pytest.mark.parametrize("case", ["grad_bucket_padded_rank_major", "grad_bucket_flat_cat", "grad_bucket_chunk_cat"])
def test_classify_copy_in_layout_reference_vectors(golden, case):
    g = golden[case]
    mps = managed(g["params"])
    bucket = MatrixGradBucket(
        tuple(BucketParamGrad(m, torch.tensor(v, dtype=torch.float32)) for m, v in zip(mps, g["grads"])),
        g["total_numel"], tuple(g["shard_sizes"]), segs(g["rank_segments"]),
    )
    assert classify_copy_in_layout(bucket) == g["layout_kind"]
    assert bucket.world_size == len(g["shard_sizes"]) and bucket.max_shard_size == max(g["shard_sizes"]) and bucket.has_grads
    # argument errors are raised before any device work (reference: grad_bucket.py:77-96)
    n = bucket.world_size * bucket.max_shard_size
    with pytest.raises(ValueError, match="1D"):
        fill_reduce_scatter_input(bucket, torch.empty(1, n))
    with pytest.raises(ValueError, match="expected"):
        fill_reduce_scatter_input(bucket, torch.empty(n + 1))
    with pytest.raises(ValueError, match="backend must be"):
        fill_reduce_scatter_input(bucket, torch.empty(n), backend="nope")
    if g["layout_kind"] != "flat_contiguous":
        with pytest.raises(ValueError, match="flat bucket layout"):
            fill_reduce_scatter_input(bucket, torch.empty(n), backend="flat_cat")
    if g["layout_kind"] != "fsdp2_chunk":
        with pytest.raises(ValueError, match="FSDP2-style"):
            fill_reduce_scatter_input(bucket, torch.empty(n), backend="chunk_cat")
    with pytest.raises(ValueError, match="at least one rank"):
        fill_reduce_scatter_input(MatrixGradBucket((), 0, (), ()), torch.empty(0))


def test_closed_form_plans():
    specs = param_specs([("a", (4, 6)), ("b", (8,))])
    plan = fsdp2_chunk_plan(specs, 2)
    assert plan.shard_sizes == (16, 16)
    assert plan.rank_segments[1] == (LayoutSegment(12, 24, 0), LayoutSegment(28, 32, 12))
    with pytest.raises(ValueError, match="divisible"):
        fsdp2_chunk_plan(param_specs([("a", (3,))]), 2)
    plan = block_grid_plan(specs, (2, 2))
    validate_shard_plan(plan)
    assert plan.shard_sizes == (8, 8, 8, 8)
    assert plan.rank_segments[3][:2] == (LayoutSegment(15, 18, 0), LayoutSegment(21, 24, 3))
    assert plan.rank_segments[3][2] == LayoutSegment(30, 32, 6)
    owner = whole_param_owner_plan(specs, 2, [1, 0])
    assert owner.shard_sizes == (8, 24) and owner.rank_segments[1] == (LayoutSegment(0, 24, 0),)
    assert rank_major_owner_order(specs, 2, [1, 0]) == [1, 0]
    assert contiguous_even_plan(7, 3).shard_sizes == (3, 2, 2)
    for w in (MLP_W2, HIDDEN2048_W4):
        validate_shard_plan(w.plan())
    assert MLP_W2.plan().shard_sizes == (131456, 131456)
    assert HIDDEN2048_W4.total_numel == 50335744 and HIDDEN4096_W4_BLOCK.total_numel == 202383360


def test_merge_runs_builds_strided_blocks():
    # R/2 row segments of C/2 elements at source pitch C, destination pitch C/2 -> one 2-D run
    rows, cols = 6, 8
    src = [r * cols + 4 for r in range(3, 6)]
    dst = [100 + k * 4 for k in range(3)]
    merged = merge_runs(make_runs(src, dst, [4, 4, 4]))
    assert merged.shape[0] == 1
    run = merged[0]
    assert (run["rows"], run["row_len"], run["src_stride"], run["dst_stride"], run["src_off"], run["dst_off"]) == (3, 4, 8, 4, 28, 100)
    # back-to-back on both sides -> one longer segment; a break in the pitch starts a new run
    assert merge_runs(make_runs([0, 4, 8], [0, 4, 8], [4, 4, 4]))[0]["row_len"] == 12
    merged = merge_runs(make_runs([0, 8, 16, 40], [0, 4, 8, 12], [4, 4, 4, 4]))
    assert [int(r["rows"]) for r in merged] == [3, 1]
    # different sources never merge
    runs = make_runs([0, 4], [0, 4], [4, 4])
    runs["src_id"] = [0, 1]
    assert merge_runs(runs).shape[0] == 2
    assert merge_runs(make_runs([], [], [])).shape[0] == 0


def test_program_create_rejects_overlapping_destination_rows():
    """The validation of ``mfsdp_segment_program_create`` runs on the host before anything touches a device: two
    interleaved column blocks of one matrix are legal (their bounding spans overlap, no row does), every true overlap
    is refused with MFSDP_ERR_INVALID.  Without a device a legal program fails later, at the upload (MFSDP_ERR_HIP)."""
    from matrix_fsdp_amd.kernels import segment_program as SP

    handle = _lib.lib()

    def create(rows):
        runs = np.zeros(len(rows), dtype=SP.RUN_DTYPE)
        for i, (src_off, dst_off, row_len, n_rows, src_stride, dst_stride) in enumerate(rows):
            runs[i] = (src_off, dst_off, row_len, n_rows, src_stride, dst_stride, 0, 0)
        numels = (ctypes.c_int64 * 1)(1 << 20)
        out = ctypes.c_void_p()
        rc = handle.mfsdp_segment_program_create(
            runs.ctypes.data_as(ctypes.POINTER(_lib.CopyRun)), len(rows), numels, 1, 1 << 20, _lib.CONVERT_NONE, 2, ctypes.byref(out)
        )
        if rc == 0:
            handle.mfsdp_segment_program_destroy(out)
        return rc, handle.mfsdp_last_error().decode()

    legal = (0, 2)  # built (a device is present) or refused by the upload only
    # left and right half of a 64 x 32 matrix as two strided runs
    assert create([(0, 0, 16, 64, 16, 32), (4096, 16, 16, 64, 16, 32)])[0] in legal
    # three runs that interleave row by row, given in any order
    assert create([(0, 20, 10, 50, 10, 30), (1000, 0, 10, 50, 10, 30), (2000, 10, 10, 50, 10, 30)])[0] in legal
    # a plain segment that starts exactly where the last row of a strided run ends
    assert create([(0, 0, 16, 64, 16, 32), (4096, 32 * 63 + 16, 17, 1, 0, 0)])[0] in legal
    # a plain segment between two rows of a strided run
    assert create([(0, 0, 16, 64, 16, 32), (4096, 16 + 32 * 7, 16, 1, 0, 0)])[0] in legal
    for rows in (
        [(0, 0, 16, 64, 16, 32), (4096, 15, 16, 64, 16, 32)],          # shifted by one element: every row overlaps
        [(0, 0, 100, 1, 0, 0), (500, 99, 5, 1, 0, 0)],                 # plain segments, one element shared
        [(0, 0, 16, 64, 16, 32), (4096, 32 * 40 + 8, 4, 1, 0, 0)],     # a short segment inside row 40
        [(0, 0, 10, 3, 10, 100), (500, 205, 10, 1, 0, 0)],             # only the last row is hit
    ):
        rc, message = create(rows)
        assert rc == 1 and "two runs write destination offset" in message, (rows, rc, message)
    # against brute force on random small programs
    rng = np.random.default_rng(0)
    seen = {True: 0, False: 0}
    for _ in range(400):
        rows, hits, clash = [], np.zeros(4096, dtype=np.int32), False
        for _ in range(int(rng.integers(2, 6))):
            row_len, n_rows = int(rng.integers(1, 12)), int(rng.integers(1, 9))
            stride = row_len + int(rng.integers(0, 20)) if n_rows > 1 else 0
            dst_off = int(rng.integers(0, 300))
            rows.append((0, dst_off, row_len, n_rows, row_len, stride))
            for r in range(n_rows):
                hits[dst_off + r * stride : dst_off + r * stride + row_len] += 1
        clash = bool((hits > 1).any())
        seen[clash] += 1
        rc, _ = create(rows)
        assert (rc == 1) == clash, (rows, rc)
    assert min(seen.values()) > 50


def test_fill_runs_cover_exactly_the_gaps():
    fills = fill_runs_for_gaps(make_runs([0, 0], [2, 8], [3, 2]), 12)
    assert [(int(f["dst_off"]), int(f["row_len"]), int(f["src_id"])) for f in fills] == [(0, 2, -1), (5, 3, -1), (10, 2, -1)]
    assert fill_runs_for_gaps(make_runs([0], [0], [12]), 12).shape[0] == 0
    with pytest.raises(ValueError, match="overlap"):
        fill_runs_for_gaps(make_runs([0, 0], [0, 2], [3, 3]), 12)


def test_grad_fill_runs_match_the_oracle_on_random_layouts():
    import random

    from tests.conftest import params_from_pairs
    from tests.test_oracle_copy import random_plan

    rng = random.Random(3)
    for _ in range(30):
        sizes = [rng.randint(1, 40) for _ in range(rng.randint(1, 6))]
        params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
        total, world = sum(sizes), rng.randint(1, 4)
        plan = random_plan(rng, total, world) if total > 1 else contiguous_even_plan(total, world)
        max_shard = plan.max_shard_size
        runs = grad_fill_runs(params, plan.rank_segments, max_shard)
        grads = [torch.arange(n, dtype=torch.float32) + 100 * (i + 1) for i, n in enumerate(sizes)]
        have = torch.zeros(world * max_shard)
        for run in runs:
            s, d, n = int(run["src_off"]), int(run["dst_off"]), int(run["row_len"])
            have[d : d + n] = grads[int(run["src_id"])][s : s + n]
        want = torch.full((world * max_shard,), -1.0)
        O.fill_reduce_scatter_input(params, grads, plan.shard_sizes, plan.rank_segments, total, want)
        assert torch.equal(have, want)


def test_fully_shard_host_rules():
    """What the lifecycle shell decides on the host: the default plan, parameter ownership of nested units, and
    that nothing runs without a HIP device (there is no CPU fallback)."""
    from matrix_fsdp_amd import MixedPrecisionPolicy, fully_shard
    from matrix_fsdp_amd.api import validate_mixed_precision_policy
    from matrix_fsdp_amd.core.managed_param import managed_params_from_module
    from matrix_fsdp_amd.runtime.param_group import default_planner

    module = torch.nn.Sequential(torch.nn.Linear(8, 4), torch.nn.Linear(4, 3))
    mps = list(managed_params_from_module(module))
    chunked = default_planner(mps, 1)
    assert chunked.shard_sizes == (sum(mp.numel for mp in mps),)
    ragged = default_planner(mps, 4)  # 3 x 4 weights and a bias of 3 do not divide by 4: rank-contiguous even split
    assert sum(ragged.shard_sizes) == mps[-1].end and max(ragged.shard_sizes) - min(ragged.shard_sizes) <= 1
    even = default_planner(mps[:2], 4)
    assert even.shard_sizes == (9, 9, 9, 9) and len(even.rank_segments[0]) == 2  # a chunk of every parameter
    with pytest.raises(RuntimeError, match="HIP device"):
        fully_shard(module)
    with pytest.raises(ValueError, match="floating-point"):
        validate_mixed_precision_policy(MixedPrecisionPolicy(reduce_dtype=torch.int64))
    # the reference's parameters come first and in its order (test/fsdp/test_matrix_fsdp_e2e.py:206-226)
    import inspect

    parameters = inspect.signature(fully_shard).parameters
    assert tuple(parameters)[:9] == ("module", "mesh", "reshard_after_forward", "shard_placement_fn", "mp_policy", "offload_policy", "ignored_params", "dp_mesh_dims", "optimizer_policy")
    assert all(parameters[name].kind == inspect.Parameter.KEYWORD_ONLY for name in tuple(parameters)[1:])
    assert parameters["reshard_after_forward"].default is None and parameters["optimizer_policy"].default is None
    from torch.distributed.fsdp import CPUOffloadPolicy

    with pytest.raises(NotImplementedError, match="CPUOffloadPolicy"):
        fully_shard(torch.nn.Linear(2, 2), offload_policy=CPUOffloadPolicy())
    with pytest.raises(TypeError, match="must be an OffloadPolicy"):
        fully_shard(torch.nn.Linear(2, 2), offload_policy="cpu")
    with pytest.raises(NotImplementedError, match="dp_mesh_dims"):
        fully_shard(torch.nn.Linear(2, 2), dp_mesh_dims=(0, 1))
    # placements other than Shard(0) are refused as in the reference (matrix_fsdp/api.py:139-149)
    from torch.distributed.tensor import Replicate, Shard

    with pytest.raises(NotImplementedError, match="only None or torch.distributed.tensor.Shard"):
        fully_shard(torch.nn.Linear(2, 2), shard_placement_fn=lambda p: Replicate())
    with pytest.raises(NotImplementedError, match="supports only Shard\\(0\\)"):
        fully_shard(torch.nn.Linear(2, 2), shard_placement_fn=lambda p: Shard(1))
    # matrix_fully_shard: switches that only steer collectives are accepted, anything unknown is not
    from matrix_fsdp_amd import matrix_fully_shard as mfs
    from matrix_fsdp_amd.core.plans import fsdp2_chunk_plan

    with pytest.raises(TypeError, match="unexpected keyword arguments: prefetch_depth"):
        mfs(torch.nn.Linear(2, 2), forward_prefetch=True, prefetch_depth=2)
    with pytest.raises(NotImplementedError, match="finalize_after_backward=False"):
        mfs(torch.nn.Linear(2, 2), finalize_after_backward=False)
    with pytest.raises(ValueError, match="either planner or group_planner"):
        mfs(torch.nn.Linear(2, 2), planner=fsdp2_chunk_plan, group_planner=fsdp2_chunk_plan)
    with pytest.raises(NotImplementedError, match="dp_shard_mesh_dim"):
        mfs(torch.nn.Linear(2, 2), dp_shard_mesh_dim=0)
    with pytest.raises(RuntimeError, match="HIP device"):  # every argument accepted: stops only at the CPU module
        mfs(torch.nn.Linear(2, 2), forward_prefetch=True, backward_prefetch=False, matrix_collective_backend="custom", group_planner=fsdp2_chunk_plan, world_size=2)
    # wrap policies decide before anything touches the device
    from matrix_fsdp_amd import matrix_fully_shard
    from matrix_fsdp_amd.policy import module_type_policy

    with pytest.raises(ValueError, match="did not select any modules"):
        matrix_fully_shard(torch.nn.Sequential(torch.nn.ReLU(), torch.nn.Tanh()), wrap_policy=module_type_policy(torch.nn.Linear))
    with pytest.raises(ValueError, match="did not select any modules"):  # selected, but all of its parameters are ignored
        lin = torch.nn.Linear(2, 2)
        matrix_fully_shard(torch.nn.Sequential(lin), wrap_policy=module_type_policy(torch.nn.Linear), ignored_params=set(lin.parameters()))
    with pytest.raises(ValueError, match="explicit shard_hints"):
        matrix_fully_shard(module, wrap_policy=module_type_policy(torch.nn.Linear), shard_hints={})
    with pytest.raises(ValueError, match="only 'muon_shard_aware'"):
        matrix_fully_shard(module, auto_planner_policy="balanced")
    with pytest.raises(ValueError, match="not both"):
        matrix_fully_shard(module, auto_planner_policy="muon_shard_aware", planner=default_planner)
    with pytest.raises(RuntimeError, match="HIP device"):
        matrix_fully_shard(module, wrap_policy=module_type_policy(torch.nn.Linear))
    with pytest.raises(NotImplementedError, match="subgroup resharding"):
        fully_shard(module, reshard_after_forward=2)
    frozen = torch.nn.Linear(2, 2)
    frozen.bias.requires_grad_(False)
    with pytest.raises(NotImplementedError, match="require grad"):
        matrix_fully_shard(frozen)


def test_wrap_policies():
    """The expectations of the reference's test/fsdp/test_wrap.py:9-65."""
    from torch import nn

    from matrix_fsdp_amd.policy import and_policy, module_type_policy, not_policy, or_policy, size_based_policy

    assert module_type_policy(nn.Linear)(nn.Linear(4, 2)) and not module_type_policy(nn.Linear)(nn.ReLU())
    both = module_type_policy({nn.Linear, nn.LayerNorm})
    assert both(nn.Linear(4, 2)) and both(nn.LayerNorm(4)) and not both(nn.ReLU())
    with pytest.raises(ValueError, match="at least one"):
        module_type_policy(set())
    with pytest.raises(TypeError, match="nn.Module types"):
        module_type_policy({nn.Linear, object})
    module = nn.Sequential(nn.Linear(4, 8), nn.ReLU(), nn.Linear(8, 2))
    assert not size_based_policy(1)(module) and size_based_policy(1)(module[0])  # own parameters only by default
    total = sum(p.numel() for p in module.parameters())
    assert size_based_policy(total, recurse=True)(module) and not size_based_policy(total + 1, recurse=True)(module)
    with pytest.raises(ValueError, match="non-negative"):
        size_based_policy(-1)
    linear, large = module_type_policy(nn.Linear), size_based_policy(32)
    assert or_policy(linear, module_type_policy(nn.LayerNorm))(nn.Linear(4, 2))
    assert not or_policy(module_type_policy(nn.LayerNorm), module_type_policy(nn.ReLU))(nn.Linear(4, 2))
    assert and_policy(linear, large)(nn.Linear(4, 8)) and not and_policy(linear, large)(nn.Linear(2, 2))
    assert not_policy(large)(nn.Linear(2, 2))
    for make in (or_policy, and_policy):
        with pytest.raises(ValueError, match="at least one"):
            make()
        with pytest.raises(TypeError, match="callable"):
            make(linear, object())
    with pytest.raises(TypeError, match="callable"):
        not_policy(object())


def test_full_param_buffer_pool_bookkeeping():
    """test/fsdp/test_flat_buffer.py:277-301 on CPU tensors with a hand-made event: a released buffer is handed
    out again only once its release event has completed; at most ``max_cached_per_key`` are held per key."""
    from matrix_fsdp_amd import FullParamBufferPool

    class Event:
        def __init__(self, complete):
            self.complete = complete

        def query(self):
            return self.complete

    pool = FullParamBufferPool(max_cached_per_key=1)
    buffer = torch.arange(6, dtype=torch.float32)
    event = Event(False)
    release = pool.release(buffer, cuda_event=event)
    assert (release.kind, release.numel, release.bytes) == ("pending_event", 6, 24)
    stats = pool.stats()
    assert (stats["cached_buffers"], stats["pending_buffers"], stats["pending_releases"], stats["pending_bytes"]) == (0, 1, 1, 24)
    assert not pool.can_cache(buffer)  # the waiting one counts
    assert pool.release(torch.zeros(6), cuda_event=Event(True)).kind == "dropped"
    fresh = pool.acquire(buffer, 6)
    assert fresh.data_ptr() != buffer.data_ptr()
    event.complete = True
    got = pool.acquire_with_stats(buffer, 6)
    assert got.reused and got.tensor.data_ptr() == buffer.data_ptr()
    stats = pool.stats()
    assert (stats["pending_buffers"], stats["reuses"], stats["allocations"], stats["drops"]) == (0, 1, 1, 1)
    # keys: device, dtype and element count
    assert pool.release(buffer).kind == "cached" and pool.release(None).kind == "none"
    assert not pool.acquire_with_stats(buffer.double(), 6).reused and not pool.acquire_with_stats(buffer, 5).reused
    assert pool.acquire_with_stats(buffer.view(2, 3), 6).reused
    pool.release(buffer)
    pool.clear()
    assert pool.stats()["cached_buffers"] == 0
    assert FullParamBufferPool().release(buffer).kind == "dropped"  # a pool of capacity 0 keeps nothing
    with pytest.raises(ValueError, match="non-negative"):
        FullParamBufferPool(max_cached_per_key=-1)
    from matrix_fsdp_amd.runtime.param_group import MatrixFSDPParamGroup

    with pytest.raises(ValueError, match="needs use_saved_tensor_hooks"):
        MatrixFSDPParamGroup(torch.nn.Linear(2, 2), full_param_buffer_pool=FullParamBufferPool(max_cached_per_key=1), use_saved_tensor_hooks=False)


def test_public_names_of_the_reference_that_this_build_provides():
    """The reference's top-level names for the path, its metadata, the lifecycle shell, the planners and the
    checkpoint format resolve on this package too (what is left out needs a process group: meshes, DTensor
    placements, collectives, the prefetch scheduler, the auto planner with its cost model)."""
    import matrix_fsdp_amd as m

    assert all(hasattr(m, name) for name in m.__all__)
    provided = """
        LayoutSegment ShardPlan MatrixGroupLayout ParamLayout ParamSegment RankLayout ManagedParam ManagedParamRegistry
        ParamShardHint ParamRuntimeKind MatrixShard PlacementCompatibility MatrixShardedState MixedPrecisionPolicy
        StaticParamBufferLayout ElasticParamBufferLayout ElasticCommunicationPlan ElasticRankChunk FullParamBufferPool
        FSDPLifecycleState MatrixFSDPParamGroup MatrixFSDPNoSync WrapPolicy
        fully_shard matrix_fully_shard configure_optimizer configure_matrix_optimizer prepare_matrix_optimizer
        install_matrix_optimizer_auto_prepare PreparedMatrixOptimizer MatrixFSDPOptimizer MixedMuonAdamWOptimizer
        MatrixOptimizerConfig MatrixOptimizerParamGroupSummary ClassifiedMatrixOptimizerParams classify_matrix_optimizer_params
        make_mixed_muon_adamw_optimizer collect_param_groups DEFAULT_MUON_ADJUST_LR_FN
        MatrixFSDPOptimizerStateManager LocalOptimizerStateTensor OptimizerStateSummary
        build_shard_hints moe_expert_owner_rule fsdp2_chunk_plan hinted_ordered_group_plan ordered_matrix_owner_tail_plan
        load_balanced_matrix_owner_tail_plan load_balanced_matrix_owner_tail_group_plans expert_owner_tail_plan
        explain_matrix_shard_compatibility is_matrix_shard_compatible_plan matrix_shard_from_plan matrix_shard_from_layout
        shard_sizes_to_matrix_local_units matrix_shard_metadata matrix_sharded_state_metadata
        explain_runtime_layout_compatibility validate_runtime_layout RuntimeLayoutCompatibility
        rank_segments_are_rank_contiguous_chunks clear_global_full_param_buffer_pool
        module_type_policy size_based_policy or_policy and_policy not_policy
        matrix_state_dict load_matrix_state_dict save_matrix_dcp load_matrix_dcp load_matrix_dcp_full_state
        get_state_dict set_state_dict get_model_state_dict set_model_state_dict get_optimizer_state_dict set_optimizer_state_dict
        patch_model_state_dict patch_optimizer_state_dict matrix_get_state_dict matrix_set_state_dict
    """.split()
    missing = [name for name in provided if not hasattr(m, name)]
    assert not missing, missing


def test_bench_refuses_more_than_one_gpu_and_the_product_has_no_cpu_path():
    """``bench.py --gpus N`` with N above 1 exits with a message before touching a device; the flat buffer refuses
    host tensors instead of falling back to host copies."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    done = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert done.returncode != 0 and "ONE GPU" in (done.stdout + done.stderr) and not done.stdout.strip().startswith("{")
    from matrix_fsdp_amd.core.managed_param import managed_params_from_module
    from matrix_fsdp_amd.core.plans import contiguous_even_plan
    from matrix_fsdp_amd.runtime.flat_buffer import MatrixFlatBuffer

    params = list(managed_params_from_module(torch.nn.Linear(4, 4)))
    with pytest.raises(RuntimeError, match="HIP device"):
        MatrixFlatBuffer(params, contiguous_even_plan(params[-1].end, 2), rank=0)


def test_mixed_optimizer_constructor_surface_of_the_reference():
    """Construction only (no step, so no device): the three cases of test/fsdp/test_bench_fsdp2_compare.py:406-424
    and the keyword set of matrix_fsdp/optim/wrapper.py:353-400."""
    from matrix_fsdp_amd.optim.wrapper import DEFAULT_MUON_ADJUST_LR_FN, MixedMuonAdamWOptimizer, _LazyMuonOptimizer

    matrix = torch.nn.Parameter(torch.ones(4, 4))
    vector = torch.nn.Parameter(torch.ones(4))
    optimizer = MixedMuonAdamWOptimizer([matrix], [])
    assert DEFAULT_MUON_ADJUST_LR_FN == "match_rms_adamw"
    assert optimizer.muon is not None and optimizer.muon.param_groups[0]["adjust_lr_fn"] == DEFAULT_MUON_ADJUST_LR_FN
    lazy = MixedMuonAdamWOptimizer([matrix], [vector], lazy_muon_init=True)
    assert lazy.muon.state == {} and lazy.state == {}
    assert lazy.muon.state_dict()["state"] == {}
    assert lazy.muon.param_groups[0]["adjust_lr_fn"] == DEFAULT_MUON_ADJUST_LR_FN
    assert isinstance(lazy.muon, _LazyMuonOptimizer) and lazy.muon.defaults["momentum"] == 0.5 and lazy.muon.defaults["ns_steps"] == 2
    matrix.grad = torch.ones(4, 4)
    lazy.zero_grad()
    assert matrix.grad is None and lazy.muon.state == {}
    matrix.grad = torch.ones(4, 4)
    lazy.muon.zero_grad(set_to_none=False)
    assert float(matrix.grad.abs().sum()) == 0.0
    every_reference_keyword = dict(
        lr=1e-3, weight_decay=0.01, muon_lr=None, adamw_lr=None, adamw_betas=(0.9, 0.999), adamw_eps=1e-8, adamw_weight_decay=None,
        adamw_foreach=None, muon_weight_decay=None, muon_momentum=0.5, muon_ns_steps=2, muon_adjust_lr_fn="match_rms_adamw",
        lazy_muon_init=False, fsdp_param_groups=None, max_unsharded_prefetch_units=None, max_forward_prefetch_units=None,
        max_backward_prefetch_units=None, backward_prefetch_timing="pre_backward", prefetch_policy="static",
        max_cached_full_param_buffers_per_key=0, max_cached_elastic_workspaces_per_key=0, max_active_full_param_buffers=None,
        max_active_full_param_numel=None, max_active_full_param_memory_mb=None, max_pending_backward_reduces=1,
        owner_backward_prefetch_with_pending_reduce="auto", trim_cuda_cache=False, cuda_cache_trim_threshold_mb=1024.0,
        flat_adamw_state=False, scheduler_config=None,
    )
    MixedMuonAdamWOptimizer([matrix], [vector], group_summaries=(), **every_reference_keyword)
    with pytest.raises(TypeError, match="unexpected keyword argument 'momentum'"):
        MixedMuonAdamWOptimizer([matrix], [], momentum=0.9)
    with pytest.raises(RuntimeError, match="at least one non-empty parameter"):
        MixedMuonAdamWOptimizer([], [])
