"""MatrixFlatBuffer on a HIP device: views alias the buffers, copies are bit-exact with the oracle."""
import pytest
import torch
from torch import nn

from matrix_fsdp_amd import LayoutSegment, ShardPlan, managed_params_from_named
from matrix_fsdp_amd.core.plans import contiguous_even_plan, fsdp2_chunk_plan, whole_param_owner_plan
from matrix_fsdp_amd.runtime.flat_buffer import MatrixFlatBuffer
from matrix_fsdp_amd.runtime.grad_bucket import (
    BucketParamGrad,
    MatrixGradBucket,
    build_reduce_scatter_input,
    classify_copy_in_layout,
    fill_reduce_scatter_input,
)
from oracle import copy_oracle as O
from tests.conftest import segs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def params(named):
    return [(n, nn.Parameter(t.to(DEV))) for n, t in named]


def test_fsdp2_chunk_buffer_reference_vectors(golden):
    g = golden["fsdp2_chunk_plan_pack_unpack"]
    named = params([("weight", torch.arange(6, dtype=torch.float32)), ("bias", torch.arange(10, 14, dtype=torch.float32))])
    mps = list(managed_params_from_named(named))
    plan = fsdp2_chunk_plan(mps, g["world_size"])
    fb = MatrixFlatBuffer(mps, plan, rank=1)
    assert fb.local_shard.cpu().tolist() == g["rank1_local_shard"]
    assert fb.local_segments == tuple(LayoutSegment(*t) for t in g["rank1_segments"])
    full = torch.tensor(g["full"], dtype=torch.float32, device=DEV)
    packed = fb._pack_full_tensor_by_rank_segments(full)
    assert packed.cpu().tolist() == g["packed"]
    assert fb._unpack_rank_shards_to_full_tensor(packed).cpu().tolist() == g["full"]
    # partial parameters are exposed as 1-D slices of the local shard
    assert fb.param_data_alias_local_shard()
    assert mps[0].param.data.shape == (3,) and mps[0].param.data.cpu().tolist() == [3, 4, 5]
    with pytest.raises(RuntimeError, match="expected"):
        fb._pack_full_tensor_by_rank_segments(full[:-1])
    with pytest.raises(RuntimeError, match="expected"):
        fb._unpack_rank_shards_to_full_tensor(packed[:-1])


def test_unpack_identity_reuses_storage_and_reordered_owners_copy(golden):
    g = golden["unpack_identity_reuses_storage"]
    named = params([("p", torch.arange(16, dtype=torch.float32))])
    fb = MatrixFlatBuffer(list(managed_params_from_named(named)), ShardPlan(16, tuple(g["shard_sizes"]), tuple(g["shard_offsets"])), rank=1)
    gathered = torch.tensor(g["gathered"], dtype=torch.float32, device=DEV)
    assert fb._unpack_rank_shards_to_full_tensor(gathered).data_ptr() == gathered.data_ptr()
    g = golden["unpack_reordered_owners"]
    named = params([("first", torch.arange(2, dtype=torch.float32)), ("second", torch.arange(10, 12, dtype=torch.float32))])
    fb = MatrixFlatBuffer(list(managed_params_from_named(named)), ShardPlan(4, (2, 2), (0, 2), segs(g["rank_segments"])), rank=0)
    packed = torch.tensor(g["packed"], dtype=torch.float32, device=DEV)
    out = fb._unpack_rank_shards_to_full_tensor(packed)
    assert out.data_ptr() != packed.data_ptr() and out.cpu().tolist() == g["full"]


def test_shard_unshard_views_alias_buffers():
    w = torch.randn(8, 6).bfloat16()
    b = torch.randn(12).bfloat16()
    named = params([("w", w), ("b", b)])
    mps = list(managed_params_from_named(named))
    fb = MatrixFlatBuffer(mps, contiguous_even_plan(60, 4), rank=2)
    assert fb.layout.padded_numel == 60 and fb.local_shard.numel() == 15
    assert fb.param_data_alias_local_shard() and not fb.param_data_alias_full_buffer()
    gathered = fb.gathered_padded_shards()
    full = fb.unshard(gathered)
    assert fb.param_data_alias_full_buffer()
    assert mps[0].param.data.shape == (8, 6) and mps[0].param.data.data_ptr() == full.data_ptr()
    assert mps[1].param.data.data_ptr() == full.data_ptr() + 48 * 2
    assert torch.equal(mps[0].param.data.cpu().view(torch.int16), w.view(torch.int16))
    assert torch.equal(mps[1].param.data.cpu().view(torch.int16), b.view(torch.int16))
    fb.use_local_shards()
    assert fb.full_buffer is None and fb.param_data_alias_local_shard()
    with pytest.raises(RuntimeError, match="not materialized"):
        fb.use_full_param_buffer()


def test_uneven_owner_layout_pads_and_packs_grads_compactly(golden):
    g = golden["compact_owner_bucket"]
    named = params([("first", torch.arange(3, dtype=torch.float32)), ("second", torch.arange(10, 11, dtype=torch.float32))])
    mps = list(managed_params_from_named(named))
    plan = ShardPlan(4, tuple(g["shard_sizes"]), (0, 3), segs(g["rank_segments"]))
    fb = MatrixFlatBuffer(mps, plan, rank=0)
    assert fb.is_whole_param_owner_layout()
    gathered = fb.gathered_padded_shards()
    assert gathered.cpu().tolist() == [0, 1, 2, 10, 0, 0]  # slot r = rank r's shard, tail zero
    assert fb.unshard(gathered).cpu().tolist() == [0, 1, 2, 10]
    # zero-copy bucket (parameters unsharded, as before backward): grads are views of the compact workspace
    assert fb.prepare_grad_bucket() and fb.grad_bucket_input_is_compact and fb.grad_bucket_input.numel() == g["compact_numel"]
    mps[0].param.grad.copy_(torch.tensor(g["grads"][0], device=DEV))
    mps[1].param.grad.copy_(torch.tensor(g["grads"][1], device=DEV))
    assert fb.grad_bucket_input.cpu().tolist() == g["compact_packed"]
    assert mps[0].param.grad.untyped_storage().data_ptr() == fb.grad_bucket_input.untyped_storage().data_ptr()
    # copy-in path
    mps[0].param.grad = torch.tensor(g["grads"][0], dtype=torch.float32, device=DEV)
    mps[1].param.grad = torch.tensor(g["grads"][1], dtype=torch.float32, device=DEV)
    bucket = fb.collect_grad_bucket()
    assert mps[0].param.grad is None
    packed = torch.full((4,), -1.0, device=DEV)
    fb._fill_compact_owner_reduce_scatter_input(bucket, packed)
    assert packed.cpu().tolist() == g["compact_packed"]
    assert fb.reduce_grad_bucket_to_local_shard(bucket).cpu().tolist() == g["rank0_local_grad_shard"]
    fb.use_local_shards()
    assert mps[1].param.data.numel() == 0  # rank 0 does not own "second"
    fb.use_local_grad_shard()
    assert mps[0].param.grad.data_ptr() == fb.local_grad_shard.data_ptr() and mps[1].param.grad is None
    with pytest.raises(ValueError, match="expected"):
        fb._fill_compact_owner_reduce_scatter_input(bucket, torch.empty(5, device=DEV))


@pytest.mark.parametrize("case", ["grad_bucket_padded_rank_major", "grad_bucket_flat_cat", "grad_bucket_chunk_cat"])
def test_grad_bucket_dispatcher_reference_vectors(golden, case):
    g = golden[case]
    named = params([(n, torch.zeros(k)) for n, k in g["params"]])
    mps = managed_params_from_named(named)
    bucket = MatrixGradBucket(
        tuple(BucketParamGrad(m, torch.tensor(v, dtype=torch.float32, device=DEV)) for m, v in zip(mps, g["grads"])),
        g["total_numel"], tuple(g["shard_sizes"]), segs(g["rank_segments"]),
    )
    assert classify_copy_in_layout(bucket) == g["layout_kind"]
    reference = torch.empty(1, device=DEV)
    assert build_reduce_scatter_input(bucket, reference).cpu().tolist() == g["packed"]
    admissible = {"flat_contiguous": ["flat_cat", "foreach_copy", "segment_copy"], "fsdp2_chunk": ["chunk_cat", "segment_copy"], "generic_segment": ["segment_copy"]}
    for backend in admissible[g["layout_kind"]]:
        packed = torch.full((len(g["packed"]),), -1.0, device=DEV)
        assert fill_reduce_scatter_input(bucket, packed, backend=backend) is packed
        assert packed.cpu().tolist() == g["packed"]
    with pytest.raises(RuntimeError, match="elements"):
        bad = MatrixGradBucket((BucketParamGrad(mps[0], torch.zeros(1, device=DEV)),) + bucket.param_grads[1:], bucket.total_numel, bucket.shard_sizes, bucket.rank_segments)
        fill_reduce_scatter_input(bad, torch.empty(len(g["packed"]), device=DEV), backend="segment_copy")


def test_mixed_precision_grad_path_row_split():
    """bf16 params and grads, fp32 reduce dtype: the copy-in widens in the same launch."""
    shapes = [("w1", (16, 8)), ("n", (8,)), ("w2", (8, 16))]
    named = params([(n, torch.randn(s).bfloat16()) for n, s in shapes])
    mps = list(managed_params_from_named(named))
    plan = fsdp2_chunk_plan(mps, 4)
    fb = MatrixFlatBuffer(mps, plan, rank=3, reduce_dtype=torch.float32)
    grads = [torch.randn(s).bfloat16() for _, s in shapes]
    fb.unshard()  # backward runs on full parameters
    for mp, gr in zip(mps, grads):
        mp.param.grad = gr.to(DEV)
    bucket = fb.collect_grad_bucket()
    fb.use_local_shards()
    assert classify_copy_in_layout(bucket) == "fsdp2_chunk"
    packed = fb.fill_reduce_scatter_input(bucket)
    assert packed.dtype == torch.float32
    expect = torch.empty(4, plan.max_shard_size)
    torch._chunk_cat([gr.reshape(-1) for gr in grads], 0, 4, out=expect)
    assert torch.equal(packed.cpu().view(torch.int32), expect.reshape(-1).view(torch.int32))
    local = fb.reduce_grad_bucket_to_local_shard(bucket)
    assert local.dtype == torch.bfloat16  # cast back to the local shard's dtype
    assert torch.equal(local.cpu().view(torch.int16), expect[3].bfloat16().view(torch.int16))
    summary = fb.communication_summary()
    assert summary["copy_in_layout_kind"] == "fsdp2_chunk" and summary["padding_waste_numel"] == 0
