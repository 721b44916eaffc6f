"""Parity of the HIP copy kernels (through the C ABI) with the CPU oracle: bit-exact."""
import random

import numpy as np
import pytest
import torch

from matrix_fsdp_amd import LayoutSegment, ShardPlan
from matrix_fsdp_amd.core.plans import block_grid_plan, contiguous_even_plan, fsdp2_chunk_plan
from matrix_fsdp_amd.kernels import native
from matrix_fsdp_amd.kernels.segment_program import (
    SegmentProgram,
    compact_owner_program,
    grad_fill_program,
    local_segments_program,
    make_runs,
    pack_program,
    unpack_program,
)
from matrix_fsdp_amd.workloads import HIDDEN2048_W4, HIDDEN4096_W4_BLOCK, MLP_W2, normal_flat, param_specs
from oracle import copy_oracle as O
from tests.conftest import params_from_pairs, segs
from tests.test_oracle_copy import random_plan

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bits(t: torch.Tensor) -> torch.Tensor:
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def assert_same_bits(have: torch.Tensor, expect: torch.Tensor):
    assert have.dtype == expect.dtype and have.shape == expect.shape
    assert torch.equal(bits(have), bits(expect))


def run_pack_unpack(plan, full_cpu, *, padded=True):
    dtype = full_cpu.dtype
    full = full_cpu.to(DEV)
    pack = pack_program(plan, dtype, padded=padded, device=DEV)
    n = len(plan.shard_sizes) * plan.max_shard_size if padded else sum(plan.shard_sizes)
    packed = torch.full((n,), 7, dtype=dtype, device=DEV)
    pack.run((full,), packed)
    expect = O.pack_to_padded(full_cpu, plan) if padded else O.pack_full_tensor_by_rank_segments(full_cpu, plan)
    assert_same_bits(packed, expect)
    unpack = unpack_program(plan, dtype, padded=padded, device=DEV)
    out = torch.full((plan.total_numel,), 9, dtype=dtype, device=DEV)
    unpack.run((packed,), out)
    assert_same_bits(out, full_cpu)
    return pack, unpack


def test_reference_vectors_pack_unpack(golden):
    g = golden["fsdp2_chunk_plan_pack_unpack"]
    plan = fsdp2_chunk_plan(params_from_pairs(g["params"]), g["world_size"])
    full = torch.tensor(g["full"], dtype=torch.float32)
    for dtype in (torch.float32, torch.bfloat16, torch.float64, torch.uint8):
        run_pack_unpack(plan, full.to(dtype), padded=False)
        run_pack_unpack(plan, full.to(dtype), padded=True)
    g = golden["unpack_reordered_owners"]
    plan = ShardPlan(g["total_numel"], tuple(g["shard_sizes"]), (0, 2), segs(g["rank_segments"]))
    out = torch.empty(4, device=DEV)
    unpack_program(plan, torch.float32, padded=False, device=DEV).run((torch.tensor(g["packed"], dtype=torch.float32, device=DEV),), out)
    assert out.cpu().tolist() == g["full"]


@pytest.mark.parametrize("case", ["grad_bucket_padded_rank_major", "grad_bucket_flat_cat", "grad_bucket_chunk_cat"])
@pytest.mark.parametrize("grad_dtype,reduce_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16)])
def test_reference_vectors_grad_copy_in(golden, case, grad_dtype, reduce_dtype):
    g = golden[case]
    params = params_from_pairs(g["params"])
    grads = [torch.tensor(v, dtype=grad_dtype, device=DEV) for v in g["grads"]]
    program = grad_fill_program(params, g["shard_sizes"], segs(g["rank_segments"]), grad_dtype, reduce_dtype, device=DEV)
    packed = torch.full((len(g["packed"]),), -1, dtype=reduce_dtype, device=DEV)
    program.run(grads, packed)
    assert_same_bits(packed, torch.tensor(g["packed"], dtype=reduce_dtype))


def test_reference_vectors_compact_owner(golden):
    g = golden["compact_owner_bucket"]
    params = params_from_pairs(g["params"])
    rank_segments = segs(g["rank_segments"])
    offsets = [O.packed_grad_offset_for_param(p, g["shard_sizes"], rank_segments, compact=True) for p in params]
    grads = [torch.tensor(v, dtype=torch.float32, device=DEV) for v in g["grads"]]
    packed = torch.full((4,), -1.0, device=DEV)
    compact_owner_program(params, offsets, 4, torch.float32, device=DEV).run(grads, packed)
    assert packed.cpu().tolist() == g["compact_packed"]
    out = torch.empty(3, device=DEV)
    with pytest.MonkeyPatch.context() as mp:
        mp.setenv("MATRIX_FSDP_ENABLE_NATIVE_COPY_KERNELS", "1")
        assert native.native_copy_rank_chunk_from_packed(packed, out, tuple(g["shard_sizes"]), 0, compact=True)
    assert out.cpu().tolist() == g["rank0_local_grad_shard"]


def test_gate_signatures_and_offset_rule(golden, monkeypatch):
    monkeypatch.delenv("MATRIX_FSDP_ENABLE_NATIVE_COPY_KERNELS", raising=False)
    src = torch.arange(6, dtype=torch.float32, device=DEV)
    out = torch.empty(4, device=DEV)
    assert not native.native_copy_rank_chunk_from_packed(src, out, (2, 4), 1, compact=True)  # opt-in
    monkeypatch.setenv("MATRIX_FSDP_ENABLE_NATIVE_COPY_KERNELS", "1")
    for case in golden["rank_chunk_offset_rule"]["cases"]:
        packed = torch.tensor(case["packed"], dtype=torch.float32, device=DEV)
        out = torch.empty(case["shard_sizes"][case["rank"]], device=DEV)
        assert native.native_copy_rank_chunk_from_packed(packed, out, tuple(case["shard_sizes"]), case["rank"], compact=case["compact"])
        if case["divide_by_world"]:
            out /= len(case["shard_sizes"])
        assert out.cpu().tolist() == case["output"]
    packed = torch.arange(8.0, device=DEV)
    out = torch.empty(2, device=DEV)
    assert native.native_copy_rank_chunk_from_packed(packed, out, (4, 2), 1, compact=False)
    assert out.cpu().tolist() == [4.0, 5.0]
    # all-gatherv self copies of the reference's two-rank tests
    for key in ("all_gatherv", "all_gatherv_fused"):
        c = golden["two_rank_collective_semantics"][key]
        full = torch.empty(len(c["output"]), device=DEV)
        for rank, rank_segs in enumerate(segs(c["rank_segments"])):
            local = torch.tensor(c["rank_shards"][rank], dtype=torch.float32, device=DEV)
            assert native.native_copy_rank_segments_to_full(local, full, rank_segs)
        assert full.cpu().tolist() == c["output"]
    # ineligible tensors -> False (caller falls back), empty segments -> True
    assert not native.native_copy_rank_segments_to_full(src.cpu(), full, (LayoutSegment(0, 1, 0),))
    assert not native.native_copy_rank_segments_to_full(src.double(), full, (LayoutSegment(0, 1, 0),))
    assert native.native_copy_rank_segments_to_full(src, full, ())


def test_error_behaviour():
    src = torch.arange(6, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="exceeds input"):
        native.copy_range(src, torch.empty(4, device=DEV), 3)
    with pytest.raises(RuntimeError, match="non-negative"):
        native.copy_range(src, torch.empty(4, device=DEV), -1)
    with pytest.raises(RuntimeError, match="dtype mismatch"):
        native.copy_range(src, torch.empty(4, device=DEV, dtype=torch.bfloat16), 0)
    native.copy_range(src, torch.empty(0, device=DEV), 6)  # empty output returns early
    with pytest.raises(RuntimeError, match="leaves"):
        SegmentProgram(make_runs([0], [3], [4]), (8,), 6, src_dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="leaves"):
        SegmentProgram(make_runs([6], [0], [4]), (8,), 6, src_dtype=torch.float32, device=DEV)
    prog = SegmentProgram(make_runs([0], [0], [4]), (8,), 6, src_dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="elements"):
        prog.run((src[:5],), torch.empty(6, device=DEV))
    with pytest.raises(RuntimeError, match="dtype"):
        prog.run((torch.empty(8, device=DEV, dtype=torch.float64),), torch.empty(6, device=DEV))
    with pytest.raises(RuntimeError, match="CUDA"):
        prog.run((torch.empty(8),), torch.empty(6, device=DEV))
    with pytest.raises(RuntimeError, match="contiguous"):
        prog.run((torch.empty(16, device=DEV)[::2],), torch.empty(6, device=DEV))


def test_copy_range_alignments():
    gen = torch.Generator().manual_seed(5)
    for dtype in (torch.uint8, torch.bfloat16, torch.float32, torch.float64):
        src_cpu = (torch.randn(5000, generator=gen) * 100).to(dtype)
        src = src_cpu.to(DEV)
        for offset, n, shift in [(0, 5000, 0), (1, 4097, 0), (3, 1, 1), (17, 1023, 3), (512, 2048, 0), (5, 0, 0)]:
            buf = torch.zeros(n + 8, dtype=dtype, device=DEV)
            out = buf[shift : shift + n]
            native.copy_range(src, out, offset)
            assert_same_bits(out, src_cpu[offset : offset + n])
            assert torch.count_nonzero(buf[:shift]) == 0 and torch.count_nonzero(buf[shift + n :]) == 0


def assert_same_bf16(have: torch.Tensor, source_f32: torch.Tensor):
    """Bit-exact with Tensor.to(bfloat16) wherever the input is a number.  NaN payloads are not
    portable (torch's own CPU conversion gives 0xFFFF from its vector loop and 0x7FC0 from its scalar
    tail), so NaN inputs must give the quiet NaN 0x7FC0 of the scalar conversion."""
    expect = source_f32.to(torch.bfloat16)
    nan = torch.isnan(source_f32)
    got = bits(have)
    assert torch.equal(got[~nan], bits(expect)[~nan])
    assert torch.all(got[nan] == 0x7FC0)


def test_cast_matches_tensor_to():
    gen = torch.Generator().manual_seed(6)
    raw = torch.randint(-(2**31), 2**31 - 1, (1 << 16,), generator=gen, dtype=torch.int64).to(torch.int32)
    special = torch.tensor([0, -(2**31), 0x7F800000, -8388608, 0x7FC00000, 0x7F800001, -1, 1, 0x8000, 0x18000, 0x3F808000, 0x3F818000, 0x7F7FFFFF], dtype=torch.int64).to(torch.int32)
    x = torch.cat((special, raw)).view(torch.float32)
    for n in (x.numel(), 13, 1, 7, 4099):
        for shift in (0, 1, 3):
            xs = x[shift : shift + n].contiguous()
            have = native.cast(xs.to(DEV)[:], torch.bfloat16)
            assert_same_bf16(have, xs)
            back = native.cast(have, torch.float32)
            assert_same_bits(back, have.cpu().to(torch.float32))
    # unaligned views
    base = x[:4100].to(DEV)
    view = base[1:4098]
    assert_same_bf16(native.cast(view, torch.bfloat16), x[1:4098])
    same = torch.ones(3, device=DEV)
    assert native.cast(same, torch.float32) is same


def test_fp16_casts_match_tensor_to():
    """float16 <-> float32: every half bit pattern widened; narrowing at every rounding boundary (each finite half
    value, the midpoint to its neighbour and one float32 step either side of it), around the overflow threshold,
    through the denormal range, and on random bit patterns.  Numbers are bit-exact against ``Tensor.to`` on the
    CPU; every NaN comes out as the quiet NaN 0x7E00 with its sign."""
    all_half = torch.arange(-(2**15), 2**15, dtype=torch.int32).to(torch.int16).view(torch.float16)
    want = all_half.to(torch.float32)
    have = native.cast(all_half.to(DEV), torch.float32).cpu()
    numbers = ~torch.isnan(want)
    assert torch.equal(have.view(torch.int32)[numbers], want.view(torch.int32)[numbers])
    assert torch.isnan(have[~numbers]).all() and int(numbers.sum()) == 65536 - 2 * 1023

    finite = want[torch.isfinite(want)].double().sort().values.unique()
    mids = ((finite[:-1] + finite[1:]) / 2).float()  # exact: 12 significant bits
    edge = torch.tensor([65504.0, 65519.99, 65520.0, 65520.01, 70000.0, 1e38, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0000001, 2.0**-26, 1e-45, 0.0])
    gen = torch.Generator().manual_seed(9)
    random_bits = torch.randint(-(2**31), 2**31 - 1, (1 << 16,), generator=gen, dtype=torch.int64).to(torch.int32).view(torch.float32)
    inf = torch.tensor(float("inf"))
    x = torch.cat((finite.float(), mids, torch.nextafter(mids, inf), torch.nextafter(mids, -inf), edge, -edge, random_bits, torch.tensor([float("inf"), float("-inf")])))
    for shift, n in ((0, x.numel()), (1, 4099), (3, 13), (0, 1)):
        xs = x[shift : shift + n].contiguous()
        have = native.cast(xs.to(DEV), torch.float16).cpu().view(torch.int16)
        want16 = xs.to(torch.float16).view(torch.int16)
        nan = torch.isnan(xs)
        assert torch.equal(have[~nan], want16[~nan])
        sign = (xs.view(torch.int32)[nan] >> 16) & -32768
        assert torch.equal(have[nan].to(torch.int32) & 0xFFFF, (sign | 0x7E00) & 0xFFFF)
    assert int(torch.isnan(x).sum()) > 0

    # the same conversions folded into segment programs: fp16 grads into an fp32 workspace, fp32 shards gathered in fp16
    rng = random.Random(3)
    for _ in range(10):
        world = rng.randint(1, 4)
        sizes = [rng.randint(1, 500) for _ in range(rng.randint(1, 5))]
        params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
        total = sum(sizes)
        plan = random_plan(rng, total, world) if total > 1 else contiguous_even_plan(total, world)
        grads_cpu = [torch.randn(n).half() for n in sizes]
        expect = torch.full((world * plan.max_shard_size,), 3.0)
        O.fill_reduce_scatter_input(params, grads_cpu, plan.shard_sizes, plan.rank_segments, total, expect)
        packed = torch.full((world * plan.max_shard_size,), 5.0, device=DEV)
        grad_fill_program(params, plan.shard_sizes, plan.rank_segments, torch.float16, torch.float32, device=DEV).run([g.to(DEV) for g in grads_cpu], packed)
        assert_same_bits(packed, expect)
        full = torch.randn(total) * 300
        gathered = torch.empty(world * plan.max_shard_size, dtype=torch.float16, device=DEV)
        pack_program(plan, torch.float32, out_dtype=torch.float16, device=DEV).run((full.to(DEV),), gathered)
        assert torch.equal(gathered.cpu().view(torch.int16), O.pack_to_padded(full, plan).to(torch.float16).view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_accumulate_matches_tensor_add(dtype):
    gen = torch.Generator().manual_seed(12)
    for n, shift in ((1 << 16, 0), (4099, 0), (4099, 1), (13, 3), (1, 0), (0, 0)):
        a = (torch.randn(n + shift, generator=gen) * 3).to(dtype)
        b = (torch.randn(n + shift, generator=gen) * 3).to(dtype)
        have = a.to(DEV)[shift:]
        have = have if shift == 0 else have  # a view that starts off the 16-byte grid when shift > 0
        out = native.accumulate(have, b.to(DEV)[shift:])
        assert out is have
        want = a[shift:].clone().add_(b[shift:])
        assert torch.equal(have.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32), want.view(torch.int16 if dtype != torch.float32 else torch.int32))
    with pytest.raises(RuntimeError, match="one dtype"):
        native.accumulate(torch.zeros(4, device=DEV), torch.zeros(4, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="elements"):
        native.accumulate(torch.zeros(4, device=DEV), torch.zeros(5, device=DEV))


def test_random_layouts_every_width():
    rng = random.Random(1)
    for trial in range(40):
        total, world = rng.randint(2, 3000), rng.randint(1, 5)
        plan = random_plan(rng, total, world)
        for dtype in (torch.bfloat16, torch.float32, torch.uint8):
            full = (torch.randperm(total) % 251 + 1).to(dtype)
            run_pack_unpack(plan, full, padded=bool(trial % 2))


def test_random_grad_copy_in_with_cast():
    rng = random.Random(2)
    for _ in range(25):
        world = rng.randint(1, 5)
        sizes = [rng.randint(1, 700) for _ in range(rng.randint(1, 6))]
        params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
        total = sum(sizes)
        plan = random_plan(rng, total, world) if total > 1 else contiguous_even_plan(total, world)
        grads_cpu = [torch.randn(n).bfloat16() for n in sizes]
        expect = torch.full((world * plan.max_shard_size,), 3.0)
        O.fill_reduce_scatter_input(params, grads_cpu, plan.shard_sizes, plan.rank_segments, total, expect)
        program = grad_fill_program(params, plan.shard_sizes, plan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
        packed = torch.full((world * plan.max_shard_size,), 5.0, device=DEV)
        program.run([g.to(DEV) for g in grads_cpu], packed)
        assert_same_bits(packed, expect)


def test_grad_copy_in_with_three_hundred_gradients():
    """fill_reduce_scatter_input takes any number of gradients (runtime/grad_bucket.py:71-116): a root unit that
    keeps what no layer manages easily holds more parameters than one launch carries pointers for."""
    rng = random.Random(3)
    world = 4
    sizes = [rng.choice([1, 7, 64, 300, 1024, 4099]) for _ in range(300)]
    params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
    total = sum(sizes)
    for plan in (contiguous_even_plan(total, world), random_plan(rng, total, world)):
        grads_cpu = [torch.randn(n, generator=torch.Generator().manual_seed(i)).bfloat16() for i, n in enumerate(sizes)]
        expect = torch.full((world * plan.max_shard_size,), 3.0)
        O.fill_reduce_scatter_input(params, grads_cpu, plan.shard_sizes, plan.rank_segments, total, expect)
        program = grad_fill_program(params, plan.shard_sizes, plan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
        packed = torch.full((world * plan.max_shard_size,), 5.0, device=DEV)
        program.run([g.to(DEV) for g in grads_cpu], packed)
        assert_same_bits(packed, expect)


def test_run_many_matches_run_buffer_by_buffer():
    """One grid over several buffers of a layout: pack, unpack and the gradient copy-in, with more buffers than one
    launch carries destinations for (64) and more source pointers than it carries (128)."""
    rng = random.Random(4)
    total, world = 5000, 3
    plan = random_plan(rng, total, world)
    pack = pack_program(plan, torch.bfloat16, device=DEV)
    unpack = unpack_program(plan, torch.bfloat16, device=DEV)
    n_buffers = 70
    fulls = [(torch.randperm(total, generator=torch.Generator().manual_seed(b)) % 251 + 1).to(torch.bfloat16) for b in range(n_buffers)]
    dev_fulls = [f.to(DEV) for f in fulls]
    padded = [torch.full((world * plan.max_shard_size,), 7, dtype=torch.bfloat16, device=DEV) for _ in range(n_buffers)]
    pack.run_many([(f,) for f in dev_fulls], padded)
    outs = [torch.full((total,), 9, dtype=torch.bfloat16, device=DEV) for _ in range(n_buffers)]
    unpack.run_many([(p,) for p in padded], outs)
    for b in range(n_buffers):
        assert_same_bits(padded[b], O.pack_to_padded(fulls[b], plan))
        assert_same_bits(outs[b], fulls[b])
    sizes = [rng.randint(1, 400) for _ in range(9)]
    params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
    gplan = random_plan(rng, sum(sizes), world)
    fill = grad_fill_program(params, gplan.shard_sizes, gplan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
    n_buffers = 20  # 180 source pointers: two launches
    grads = [[torch.randn(n, generator=torch.Generator().manual_seed(100 * b + i)).bfloat16() for i, n in enumerate(sizes)] for b in range(n_buffers)]
    packed = [torch.full((world * gplan.max_shard_size,), 5.0, device=DEV) for _ in range(n_buffers)]
    fill.run_many([[g.to(DEV) for g in gs] for gs in grads], packed)
    for b in range(n_buffers):
        expect = torch.full((world * gplan.max_shard_size,), 3.0)
        O.fill_reduce_scatter_input(params, grads[b], gplan.shard_sizes, gplan.rank_segments, sum(sizes), expect)
        assert_same_bits(packed[b], expect)
    with pytest.raises(RuntimeError, match="source lists"):
        pack.run_many([(dev_fulls[0],)], padded[:2])


def test_base_pointers_less_aligned_than_the_layout_run_the_same_tables():
    """A program compiled for 16-byte groups replayed on views that start 2, 4, 6, ... bytes into their allocations
    (narrower vector width, same tables: no table is built at run time), for plain copies and for the widening and
    narrowing conversions."""
    w = MLP_W2
    plan = w.plan()
    full = normal_flat(w.total_numel, 0.02, 5, torch.bfloat16)
    want_padded = O.pack_to_padded(full, plan)
    pack = pack_program(plan, torch.bfloat16, device=DEV)
    unpack = unpack_program(plan, torch.bfloat16, device=DEV)
    n_padded = w.world_size * plan.max_shard_size
    for src_shift, dst_shift in ((0, 0), (1, 0), (0, 1), (2, 4), (3, 5), (4, 4), (7, 1)):
        src = torch.zeros(w.total_numel + src_shift, dtype=torch.bfloat16, device=DEV)[src_shift:]
        src.copy_(full)
        guard = torch.full((n_padded + dst_shift + 8,), 3, dtype=torch.bfloat16, device=DEV)
        dst = guard[dst_shift : dst_shift + n_padded]
        free_before = torch.cuda.mem_get_info()[0]
        pack.run((src,), dst)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert_same_bits(dst, want_padded)
        assert bool((guard[:dst_shift] == 3).all()) and bool((guard[dst_shift + n_padded :] == 3).all())
        back = torch.zeros(w.total_numel + src_shift, dtype=torch.bfloat16, device=DEV)[src_shift:]
        unpack.run((dst,), back)
        assert_same_bits(back, full)
    fill = grad_fill_program(w.specs, plan.shard_sizes, plan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
    grads_cpu = [normal_flat(s.numel, 1e-3, 6 + i, torch.bfloat16) for i, s in enumerate(w.specs)]
    expect = torch.full((n_padded,), 3.0)
    O.fill_reduce_scatter_input(w.specs, grads_cpu, plan.shard_sizes, plan.rank_segments, w.total_numel, expect)
    for shift in (0, 1, 2, 3):
        grads = []
        for g in grads_cpu:
            holder = torch.zeros(g.numel() + shift, dtype=torch.bfloat16, device=DEV)[shift:]
            holder.copy_(g)
            grads.append(holder)
        packed = torch.full((n_padded + shift,), 5.0, device=DEV)[shift:]
        fill.run(grads, packed)
        assert_same_bits(packed, expect)


@pytest.mark.parametrize("world", [2, 3, 4])
def test_chunk_cat_with_ragged_params(world):
    sizes = [5, 6, 1, 16, 33, world, 3 * world + 1, 4096 + 3]
    params = params_from_pairs([(f"p{i}", n) for i, n in enumerate(sizes)])
    # the fsdp2-style layout with ceil(n/W) chunks, as _can_use_chunk_cat_fast_path expects it
    rank_segments, local = [[] for _ in range(world)], 0
    for p in params:
        chunk = -(-p.numel // world)
        for r in range(world):
            a, b = p.offset + r * chunk, min(p.end, p.offset + (r + 1) * chunk)
            if a < b:
                rank_segments[r].append(LayoutSegment(a, b, local))
        local += chunk
    shard_sizes = (local,) * world
    grads_cpu = [torch.randn(n).bfloat16() for n in sizes]
    assert O.classify_copy_in_layout(params, grads_cpu, shard_sizes, rank_segments, sum(sizes)) == "fsdp2_chunk"
    expect = torch.empty(world, local)
    torch._chunk_cat(grads_cpu, 0, world, out=expect)
    program = grad_fill_program(params, shard_sizes, rank_segments, torch.bfloat16, torch.float32, device=DEV)
    packed = torch.full((world * local,), 5.0, device=DEV)
    program.run([g.to(DEV) for g in grads_cpu], packed)
    assert_same_bits(packed.view(world, local), expect)


def test_empty_and_degenerate():
    plan = ShardPlan(0, (0, 0), (0, 0))
    pack_program(plan, torch.bfloat16, device=DEV).run((torch.empty(0, dtype=torch.bfloat16, device=DEV),), torch.empty(0, dtype=torch.bfloat16, device=DEV))
    plan = ShardPlan.from_rank_segments(5, ((LayoutSegment(0, 5, 0),), (), ()))
    run_pack_unpack(plan, torch.arange(5, dtype=torch.float32) + 1)
    run_pack_unpack(contiguous_even_plan(7, 1), torch.arange(7, dtype=torch.float32) + 1)


def test_mlp_w2_bit_exact():
    """4 bf16 params (512x256, 256, 256x512, 512), N(0, 0.02), seed 0, row-sharded for W=2."""
    w = MLP_W2
    full = normal_flat(w.total_numel, 0.02, w.seed, torch.bfloat16)
    plan = w.plan()
    assert plan.shard_sizes == (131456, 131456)
    _, unpack = run_pack_unpack(plan, full)
    out = torch.empty(w.total_numel, dtype=torch.bfloat16, device=DEV)
    unpack.run((O.pack_to_padded(full, plan).to(DEV),), out)
    for spec, view in zip(w.specs, O.param_views(out, w.specs)):
        assert view.shape == spec.shape and view.data_ptr() == out.data_ptr() + 2 * spec.offset
        assert_same_bits(view, full[spec.offset : spec.end].view(spec.shape))


def test_hidden2048_layer_pack_unpack_chunk_cat():
    w = HIDDEN2048_W4
    plan = w.plan()
    full = normal_flat(w.total_numel, 0.02, w.seed, torch.bfloat16)
    pack, unpack = run_pack_unpack(plan, full)
    assert pack.bytes_moved == 4 * w.total_numel and unpack.bytes_moved == 4 * w.total_numel
    assert pack.num_runs <= 4 * len(w.specs)
    grads_cpu = [normal_flat(s.numel, 1e-3, w.grad_seed + i, torch.bfloat16) for i, s in enumerate(w.specs)]
    expect = torch.empty(w.world_size, plan.max_shard_size)
    torch._chunk_cat(grads_cpu, 0, w.world_size, out=expect)
    program = grad_fill_program(w.specs, plan.shard_sizes, plan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
    assert program.bytes_moved == 6 * w.total_numel
    packed = torch.full((w.world_size * plan.max_shard_size,), 5.0, device=DEV)
    program.run([g.to(DEV) for g in grads_cpu], packed)
    assert_same_bits(packed.view(w.world_size, -1), expect)
    for r in range(w.world_size):  # row r = concat of every grad's r-th row block, widened
        assert_same_bits(packed.view(w.world_size, -1)[r], torch.cat([g.view(w.world_size, -1)[r] for g in grads_cpu]).float())


def test_hidden4096_block_layer_strided_pack_unpack():
    w = HIDDEN4096_W4_BLOCK
    plan = w.plan()
    assert sum(len(s) for s in plan.rank_segments) > 80000
    full = normal_flat(w.total_numel, 0.02, w.seed, torch.bfloat16)
    dev_full = full.to(DEV)
    pack = pack_program(plan, torch.bfloat16, device=DEV)
    assert pack.num_runs <= 4 * len(w.specs)  # at most one strided run per (parameter, rank)
    packed = torch.empty(4 * plan.max_shard_size, dtype=torch.bfloat16, device=DEV)
    pack.run((dev_full,), packed)
    # closed form: rank (i, j) holds the contiguous copy of each matrix's block (i, j)
    for r in range(4):
        i, j = divmod(r, 2)
        pieces = []
        for s in w.specs:
            t = full[s.offset : s.end]
            if len(s.shape) == 2:
                rows, cols = s.shape
                pieces.append(t.view(rows, cols)[i * rows // 2 : (i + 1) * rows // 2, j * cols // 2 : (j + 1) * cols // 2].reshape(-1))
            else:
                q = s.numel // 4
                pieces.append(t[r * q : (r + 1) * q])
        assert_same_bits(packed[r * plan.max_shard_size : (r + 1) * plan.max_shard_size], torch.cat(pieces))
    out = torch.empty(w.total_numel, dtype=torch.bfloat16, device=DEV)
    unpack_program(plan, torch.bfloat16, device=DEV).run((packed,), out)
    assert_same_bits(out, full)


def test_uncached_segment_copy_entry_point():
    import ctypes

    from matrix_fsdp_amd import _lib

    local = torch.arange(10, dtype=torch.float32, device=DEV)
    out = torch.zeros(12, device=DEV)
    arr = lambda v: (ctypes.c_int64 * len(v))(*v)
    torch.cuda.synchronize()
    _lib.check(_lib.lib().mfsdp_copy_rank_segments_to_full(local.data_ptr(), 10, out.data_ptr(), 12, arr([8, 0]), arr([0, 4]), arr([4, 6]), 2, 4, None))
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [4, 5, 6, 7, 8, 9, 0, 0, 0, 1, 2, 3]
    assert _lib.lib().mfsdp_copy_rank_segments_to_full(local.data_ptr(), 10, out.data_ptr(), 12, arr([9]), arr([0]), arr([4]), 1, 4, None) != 0
