"""Pins the CPU copy oracle: the reference's own literal vectors, the library
routine torch._chunk_cat, strided-slice closed forms, and invariants."""
import random

import pytest
import torch

from matrix_fsdp_amd import LayoutSegment, ShardPlan
from matrix_fsdp_amd.core.plans import block_grid_plan, contiguous_even_plan, fsdp2_chunk_plan
from matrix_fsdp_amd.workloads import param_specs
from oracle import copy_oracle as O
from tests.conftest import params_from_pairs, segs


def f32(values):
    return torch.tensor(values, dtype=torch.float32)


@pytest.mark.parametrize("case", ["grad_bucket_padded_rank_major", "grad_bucket_flat_cat", "grad_bucket_chunk_cat"])
def test_fill_reduce_scatter_input_reference_vectors(golden, case):
    g = golden[case]
    params = params_from_pairs(g["params"])
    grads = [f32(v) for v in g["grads"]]
    rank_segments = segs(g["rank_segments"])
    assert O.classify_copy_in_layout(params, grads, g["shard_sizes"], rank_segments, g["total_numel"]) == g["layout_kind"]
    packed = torch.full((len(g["shard_sizes"]) * max(g["shard_sizes"]),), -7.0)
    O.fill_reduce_scatter_input(params, grads, g["shard_sizes"], rank_segments, g["total_numel"], packed)
    assert torch.equal(packed, f32(g["packed"]))
    # every explicit backend the layout admits gives the same bytes (reference: :478-506, :535-545)
    backends = {"flat_contiguous": ["flat_cat", "foreach_copy", "segment_copy"], "fsdp2_chunk": ["chunk_cat", "segment_copy"], "generic_segment": ["segment_copy"]}
    for backend in backends[g["layout_kind"]]:
        other = torch.full_like(packed, -3.0)
        O.fill_reduce_scatter_input(params, grads, g["shard_sizes"], rank_segments, g["total_numel"], other, backend=backend)
        assert torch.equal(other, packed), backend


def test_fill_rejects_backends_the_layout_does_not_admit(golden):
    g = golden["grad_bucket_padded_rank_major"]
    params = params_from_pairs(g["params"])
    grads = [f32(v) for v in g["grads"]]
    packed = torch.empty(12)
    for backend in ("flat_cat", "foreach_copy", "chunk_cat"):
        with pytest.raises(ValueError):
            O.fill_reduce_scatter_input(params, grads, g["shard_sizes"], segs(g["rank_segments"]), 10, packed, backend=backend)
    with pytest.raises(ValueError):
        O.fill_reduce_scatter_input(params, grads, g["shard_sizes"], segs(g["rank_segments"]), 10, torch.empty(11))
    with pytest.raises(ValueError):
        O.fill_reduce_scatter_input(params, grads, g["shard_sizes"], segs(g["rank_segments"]), 10, torch.empty(3, 4))


def test_fsdp2_chunk_plan_pack_unpack_reference_vectors(golden):
    g = golden["fsdp2_chunk_plan_pack_unpack"]
    params = params_from_pairs(g["params"])
    plan = fsdp2_chunk_plan(params, g["world_size"])
    assert plan.local_segments(1) == tuple(LayoutSegment(*t) for t in g["rank1_segments"])
    full = f32(g["full"])
    packed = O.pack_full_tensor_by_rank_segments(full, plan)
    assert torch.equal(packed, f32(g["packed"]))
    start, end = plan.rank_packed_offset(1), plan.rank_packed_offset(1) + plan.shard_sizes[1]
    assert torch.equal(packed[start:end], f32(g["rank1_local_shard"]))
    assert torch.equal(O.unpack_rank_shards_to_full_tensor(packed, plan), full)


def test_unpack_identity_reuses_storage(golden):
    g = golden["unpack_identity_reuses_storage"]
    plan = ShardPlan(g["total_numel"], tuple(g["shard_sizes"]), tuple(g["shard_offsets"]))
    gathered = f32(g["gathered"])
    out = O.unpack_rank_shards_to_full_tensor(gathered, plan)
    assert out.data_ptr() == gathered.data_ptr()
    assert O.packed_rank_shards_are_full_tensor_order(plan)


def test_unpack_reordered_owners(golden):
    g = golden["unpack_reordered_owners"]
    plan = ShardPlan(g["total_numel"], tuple(g["shard_sizes"]), (0, 2), segs(g["rank_segments"]))
    packed = f32(g["packed"])
    out = O.unpack_rank_shards_to_full_tensor(packed, plan)
    assert out.data_ptr() != packed.data_ptr()
    assert torch.equal(out, f32(g["full"]))
    assert not O.packed_rank_shards_are_full_tensor_order(plan)


def test_compact_owner_bucket(golden):
    g = golden["compact_owner_bucket"]
    params = params_from_pairs(g["params"])
    grads = [f32(v) for v in g["grads"]]
    rank_segments = segs(g["rank_segments"])
    packed = torch.full((g["compact_numel"],), 9.0)
    O.fill_compact_owner_reduce_scatter_input(params, grads, g["shard_sizes"], rank_segments, packed)
    assert torch.equal(packed, f32(g["compact_packed"]))
    assert len(g["shard_sizes"]) * max(g["shard_sizes"]) == g["padded_numel"]
    out = torch.empty(g["shard_sizes"][0])
    O.copy_rank_chunk_from_packed(packed, out, g["shard_sizes"], 0, compact=True)
    assert torch.equal(out, f32(g["rank0_local_grad_shard"]))
    with pytest.raises(ValueError):
        O.fill_compact_owner_reduce_scatter_input(params, grads, g["shard_sizes"], rank_segments, torch.empty(5))


def test_rank_chunk_offset_rule(golden):
    for case in golden["rank_chunk_offset_rule"]["cases"]:
        packed = f32(case["packed"])
        out = torch.empty(case["shard_sizes"][case["rank"]])
        O.copy_rank_chunk_from_packed(packed, out, case["shard_sizes"], case["rank"], compact=case["compact"])
        if case["divide_by_world"]:
            out /= len(case["shard_sizes"])
        assert torch.equal(out, f32(case["output"]))
    # padded rule: offset = rank * max(shard_sizes)
    packed = torch.arange(8.0)
    out = torch.empty(2)
    O.copy_rank_chunk_from_packed(packed, out, (4, 2), 1, compact=False)
    assert torch.equal(out, f32([4, 5]))


def test_two_rank_gather_and_reduce_semantics(golden):
    g = golden["two_rank_collective_semantics"]
    for key in ("all_gatherv", "all_gatherv_fused"):
        c = g[key]
        out = torch.empty(len(c["output"]))
        for rank, rank_segs in enumerate(segs(c["rank_segments"])):
            O.copy_local_rank_segments(f32(c["rank_shards"][rank]), out, rank_segs)
        assert torch.equal(out, f32(c["output"]))
    c = g["reduce_scatterv"]
    total = sum(f32(v) for v in c["rank_inputs"])
    for rank, expect in enumerate(c["rank_outputs"]):
        out = torch.empty(c["shard_sizes"][rank])
        O.copy_rank_chunk_from_packed(total, out, c["shard_sizes"], rank, compact=True)
        assert torch.equal(out / 2, f32(expect))


def test_kernel_form_of_the_rank_segment_copy_against_a_literal_grid_walk():
    """``copy_rank_segments_to_full_kernel``: every (block, thread) of the reference's launch
    (matrix_copy_cuda.cu:8-23, 45-51) visited one by one on small inputs."""
    gen = torch.Generator().manual_seed(5)
    for trial in range(12):
        n_seg = int(torch.randint(1, 6, (1,), generator=gen))
        numels = [int(torch.randint(0, 700, (1,), generator=gen)) for _ in range(n_seg)]
        local_starts, cursor = [], 0
        for n in numels:
            local_starts.append(cursor)
            cursor += n
        order = torch.randperm(n_seg, generator=gen).tolist()
        global_starts, gcursor = [0] * n_seg, 3
        for i in order:
            global_starts[i] = gcursor
            gcursor += numels[i] + 2
        local = torch.arange(cursor, dtype=torch.float32) + 1
        max_numel = max(numels) if trial % 3 else max(numels) // 2  # every third trial: a max_numel that is too small
        want = torch.zeros(gcursor)
        threads, tiles = 256, (max_numel + 255) // 256
        for segment in range(n_seg):  # blockIdx.y
            for block in range(tiles):  # blockIdx.x
                for thread in range(threads):
                    offset = block * threads + thread
                    if offset < numels[segment]:
                        want[global_starts[segment] + offset] = local[local_starts[segment] + offset]
        have = torch.zeros(gcursor)
        O.copy_rank_segments_to_full_kernel(local, have, global_starts, local_starts, numels, max_numel)
        assert torch.equal(have, want)
        if max_numel >= max(numels):
            via_slices = torch.zeros(gcursor)
            O.copy_local_rank_segments(local, via_slices, segs([[(g, g + n, l) for g, l, n in zip(global_starts, local_starts, numels)]])[0])
            assert torch.equal(have, via_slices)


def test_padded_gather_and_unpad():
    sizes = (4, 6, 0, 3)
    shards = [torch.arange(n, dtype=torch.float32) + 10 * r for r, n in enumerate(sizes)]
    gathered = O.gather_padded(shards, sizes)
    assert gathered.numel() == 4 * 6
    for r, n in enumerate(sizes):
        assert torch.equal(gathered[r * 6 : r * 6 + n], shards[r])
        assert torch.count_nonzero(gathered[r * 6 + n : (r + 1) * 6]) == 0
    assert torch.equal(O.unpad_gathered(gathered, sizes), torch.cat(shards))


@pytest.mark.parametrize("world", [1, 2, 3, 4, 7])
def test_chunk_cat_matches_library_routine(world):
    """torch._chunk_cat is the routine the reference calls (grad_bucket.py:200-202)."""
    gen = torch.Generator().manual_seed(world)
    sizes = [5, 6, 1, 16, 33, world, world * 3 + 1]
    grads = [torch.randn(n, generator=gen).bfloat16() for n in sizes]
    width = sum(-(-n // world) for n in sizes)
    for dtype in (torch.bfloat16, torch.float32):
        expect = torch.full((world, width), 5.0, dtype=dtype)
        torch._chunk_cat(grads, 0, world, out=expect)
        have = torch.full((world, width), -5.0, dtype=dtype)
        O.chunk_cat([O.maybe_cast(g, dtype) for g in grads], world, have)
        assert torch.equal(have, expect)


def test_chunk_cat_row_is_concat_of_param_rows():
    """Row r of the copy-in equals cat_p(grad_p.view(W, -1)[r]) when W divides every param."""
    world = 4
    specs = param_specs([("a", (8, 6)), ("b", (12,)), ("c", (4, 4))])
    plan = fsdp2_chunk_plan(specs, world)
    grads = [torch.randn(s.numel).bfloat16() for s in specs]
    packed = torch.empty(world * plan.max_shard_size, dtype=torch.float32)
    O.fill_reduce_scatter_input(specs, grads, plan.shard_sizes, plan.rank_segments, plan.total_numel, packed)
    assert O.classify_copy_in_layout(specs, grads, plan.shard_sizes, plan.rank_segments, plan.total_numel) == "fsdp2_chunk"
    for r in range(world):
        expect = torch.cat([g.view(world, -1)[r] for g in grads]).float()
        assert torch.equal(packed.view(world, -1)[r], expect)


def test_block_grid_layout_matches_strided_slices():
    specs = param_specs([("w", (8, 12)), ("v", (16,)), ("u", (6, 4))])
    plan = block_grid_plan(specs, (2, 2))
    full = torch.arange(plan.total_numel, dtype=torch.float32)
    packed = O.pack_full_tensor_by_rank_segments(full, plan)
    for r in range(4):
        i, j = divmod(r, 2)
        pieces = []
        for s in specs:
            t = full[s.offset : s.end]
            if len(s.shape) == 2:
                rows, cols = s.shape
                pieces.append(t.view(rows, cols)[i * rows // 2 : (i + 1) * rows // 2, j * cols // 2 : (j + 1) * cols // 2].reshape(-1))
            else:
                q = s.numel // 4
                pieces.append(t[r * q : (r + 1) * q])
        start = plan.rank_packed_offset(r)
        assert torch.equal(packed[start : start + plan.shard_sizes[r]], torch.cat(pieces))
    assert torch.equal(O.unpack_rank_shards_to_full_tensor(packed, plan), full)


def random_plan(rng: random.Random, total: int, world: int) -> ShardPlan:
    """Random cover of [0, total) by segments dealt to random ranks."""
    cuts = sorted(rng.sample(range(1, total), min(total - 1, rng.randint(0, 12))))
    bounds = [0, *cuts, total]
    rank_lists = [[] for _ in range(world)]
    pieces = list(zip(bounds[:-1], bounds[1:]))
    rng.shuffle(pieces)
    for a, b in pieces:
        rank_lists[rng.randrange(world)].append((a, b))
    rank_segments = []
    for pieces_r in rank_lists:
        local, out = 0, []
        for a, b in pieces_r:
            out.append(LayoutSegment(a, b, local))
            local += b - a
        rank_segments.append(tuple(out))
    return ShardPlan.from_rank_segments(total, rank_segments)


def test_round_trip_and_write_once_on_random_layouts():
    rng = random.Random(0)
    for _ in range(50):
        total, world = rng.randint(2, 200), rng.randint(1, 5)
        plan = random_plan(rng, total, world)
        full = torch.randperm(total).float() + 1  # all distinct, non-zero
        padded = O.pack_to_padded(full, plan)
        assert padded.numel() == world * plan.max_shard_size
        assert sorted(padded[padded != 0].tolist()) == sorted(full.tolist())  # each element exactly once, rest zero
        assert torch.equal(O.unpack_from_padded(padded, plan), full)


def test_checkpoint_redistribution_on_random_layouts():
    """A rank's shard of the full buffer is that rank's slice of the packed order; the reference's
    concatenation of source shards is the full buffer exactly when the layout is rank-ordered, and the unpack is in
    every case; a parameter's local part is the matching piece of the rank's shard."""
    rng = random.Random(1)
    ordered = 0
    for _ in range(60):
        total, world = rng.randint(2, 200), rng.randint(1, 5)
        plan = random_plan(rng, total, world) if rng.random() < 0.7 else contiguous_even_plan(total, world)
        full = torch.randperm(total).float() + 1
        packed = O.pack_full_tensor_by_rank_segments(full, plan)
        shards = []
        for rank in range(world):
            start = O.rank_packed_offset(plan.shard_sizes, rank)
            shard = O.target_local_shard_from_full(full, plan.rank_segments[rank])
            assert torch.equal(shard, packed[start : start + plan.shard_sizes[rank]])
            shards.append(shard)
        joined = O.full_from_source_rank_shards(shards)
        assert torch.equal(joined, packed)
        assert torch.equal(joined, full) == O.packed_rank_shards_are_full_tensor_order(plan)
        ordered += int(torch.equal(joined, full))
        assert torch.equal(O.unpack_rank_shards_to_full_tensor(joined, plan), full)
        # a "parameter" [a, b) of the flat buffer and a moment tensor over it
        a = rng.randint(0, total - 1)
        b = rng.randint(a + 1, total)
        moment = full[a:b] * 2
        for rank in range(world):
            pieces = [type(seg)(max(a, seg.global_start), min(b, seg.global_end), 0) for seg in plan.rank_segments[rank] if max(a, seg.global_start) < min(b, seg.global_end)]
            local = O.target_local_param_tensor_from_full(moment, pieces, a)
            want = torch.cat([shards[rank][seg.local_start + max(a, seg.global_start) - seg.global_start : seg.local_start + min(b, seg.global_end) - seg.global_start] for seg in plan.rank_segments[rank] if max(a, seg.global_start) < min(b, seg.global_end)] or [full.new_empty(0)])
            assert torch.equal(local, want * 2)
    assert 0 < ordered < 60  # both kinds of layout occurred


def test_even_plan_sizes():
    plan = contiguous_even_plan(10, 4)
    assert plan.shard_sizes == (3, 3, 2, 2) and plan.shard_offsets == (0, 3, 6, 8)
    assert O.packed_rank_shards_are_full_tensor_order(plan)


def test_casts_match_tensor_to():
    bits = torch.tensor(
        [0x00000000, 0x80000000, 0x3F800000, 0x3F808000, 0x3F818000, 0x3F80FFFF, 0x7F7FFFFF, 0x7F800000, 0xFF800000,
         0x7FC00000, 0x7F800001, 0xFFFFFFFF, 0x00000001, 0x00008000, 0x00018000, 0x807FFFFF],
        dtype=torch.int64,
    ).to(torch.int32)
    x = bits.view(torch.float32)
    down = O.maybe_cast(x, torch.bfloat16)
    assert down.dtype == torch.bfloat16
    # hand-computed RNE results for the non-NaN patterns
    expect = [0x0000, 0x8000, 0x3F80, 0x3F80, 0x3F82, 0x3F81, 0x7F80, 0x7F80, 0xFF80]
    assert (down.view(torch.int16)[:9].to(torch.int32) & 0xFFFF).tolist() == expect
    assert torch.isnan(down[9:12].float()).all()
    up = O.maybe_cast(down, torch.float32)
    assert torch.equal(up.view(torch.int32)[:9], (down.view(torch.int16)[:9].to(torch.int32) << 16))
    assert O.maybe_cast(x, None) is x and O.maybe_cast(x, torch.float32) is x
    ints = torch.arange(4)
    assert O.maybe_cast(ints, torch.bfloat16) is ints
