"""The rank-segment copy with DEVICE metadata (the reference extension's own contract, matrix_copy.cpp:53-83) through
the C ABI: bit-exact against the CPU oracle for every element size, alignment and launch shape, the reference's
error cases, metadata the kernel must refuse, and replays under HIP graph capture."""
import numpy as np
import pytest
import torch

from matrix_fsdp_amd import LayoutSegment
from matrix_fsdp_amd.kernels import native as N
from matrix_fsdp_amd.kernels.segment_program import local_segments_program
from matrix_fsdp_amd.workloads import HIDDEN4096_W4_BLOCK
from oracle import copy_oracle as CO
from tests.test_copy_gpu import assert_same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.uint8, torch.bfloat16, torch.float32, torch.float64]


def random_values(n, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    if dtype == torch.uint8:
        return torch.randint(0, 256, (n,), dtype=torch.uint8, generator=gen)
    return (torch.randn(n, generator=gen) * 3).to(dtype)


def random_segments(rng, n_seg, max_len, *, lengths=None):
    """Disjoint segments: consecutive in the local shard (with gaps), shuffled in the output (with gaps)."""
    lengths = lengths if lengths is not None else [int(rng.integers(0, max_len + 1)) for _ in range(n_seg)]
    local_starts, cursor = [], int(rng.integers(0, 5))
    for n in lengths:
        local_starts.append(cursor)
        cursor += n + int(rng.integers(0, 4))
    global_starts, gcursor = [0] * len(lengths), int(rng.integers(0, 5))
    for i in rng.permutation(len(lengths)):
        global_starts[i] = gcursor
        gcursor += lengths[i] + int(rng.integers(0, 4))
    return global_starts, local_starts, lengths, cursor, gcursor


def run_device(local, output, gs, ls, ln, max_numel, balanced):
    meta = [torch.tensor(v, dtype=torch.int64, device=DEV) for v in (gs, ls, ln)]
    ws = N.copy_rank_segments_workspace(len(gs), DEV) if balanced else None
    N.copy_rank_segments_to_full(local, output, *meta, max_numel, workspace=ws)


@pytest.mark.parametrize("balanced", [False, True], ids=["uniform", "balanced"])
def test_reference_vector_reordered_owners(golden, balanced):
    """[20, 21, 10, 11] -> [10, 11, 20, 21] (reference test/fsdp/test_flat_buffer.py:603-622)."""
    local = torch.tensor([20.0, 21.0, 10.0, 11.0], device=DEV)
    out = torch.zeros(4, device=DEV)
    run_device(local, out, [2, 0], [0, 2], [2, 2], 2, balanced)
    assert out.tolist() == [10.0, 11.0, 20.0, 21.0]


@pytest.mark.parametrize("balanced", [False, True], ids=["uniform", "balanced"])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
def test_random_layouts_every_alignment(dtype, balanced):
    rng = np.random.default_rng(7)
    for trial in range(12):
        n_seg = int(rng.integers(1, 40))
        gs, ls, ln, local_n, out_n = random_segments(rng, n_seg, [9, 300, 5000][trial % 3])
        # views at odd element offsets: base pointers of every alignment the dtype allows
        shift_l, shift_o = int(rng.integers(0, 9)), int(rng.integers(0, 9))
        host_local = random_values(local_n + shift_l, dtype, 100 + trial)
        host_out = random_values(out_n + shift_o, dtype, 200 + trial)
        local, out = host_local.to(DEV)[shift_l:], host_out.to(DEV)[shift_o:]
        want = host_out[shift_o:].clone()
        CO.copy_rank_segments_to_full_kernel(host_local[shift_l:], want, gs, ls, ln, max(ln))
        run_device(local, out, gs, ls, ln, max(ln), balanced)
        assert_same_bits(out, want)


@pytest.mark.parametrize("balanced", [False, True], ids=["uniform", "balanced"])
def test_one_long_segment_beside_many_short_ones(balanced):
    rng = np.random.default_rng(3)
    lengths = [int(rng.integers(1, 64)) for _ in range(300)]
    lengths[117] = 3_000_001
    gs, ls, ln, local_n, out_n = random_segments(rng, len(lengths), 0, lengths=lengths)
    host_local, host_out = random_values(local_n, torch.bfloat16, 1), random_values(out_n, torch.bfloat16, 2)
    want = host_out.clone()
    CO.copy_rank_segments_to_full_kernel(host_local, want, gs, ls, ln, max(ln))
    out = host_out.to(DEV)
    run_device(host_local.to(DEV), out, gs, ls, ln, max(ln), balanced)
    assert_same_bits(out, want)


@pytest.mark.parametrize("n_seg", [1023, 1024, 1025, 2048, 3333])
def test_segment_counts_around_the_blocks_of_the_tile_count_tables(n_seg):
    """The balanced shape keeps its running tile counts per block of 1024 segments plus one offset per block: segment
    counts just below, at and above the block size, with empty segments and one long segment in the last block."""
    rng = np.random.default_rng(n_seg)
    lengths = [int(rng.integers(0, 700)) if rng.integers(0, 5) else 0 for _ in range(n_seg)]
    lengths[-1] = 40_000
    lengths[n_seg // 2] = 0
    gs, ls, ln, local_n, out_n = random_segments(rng, n_seg, 0, lengths=lengths)
    host_local, host_out = random_values(local_n, torch.bfloat16, 5), random_values(out_n, torch.bfloat16, 6)
    want = host_out.clone()
    CO.copy_rank_segments_to_full_kernel(host_local, want, gs, ls, ln, max(ln))
    out = host_out.to(DEV)
    run_device(host_local.to(DEV), out, gs, ls, ln, max(ln), True)
    assert_same_bits(out, want)


@pytest.mark.parametrize("balanced", [False, True], ids=["uniform", "balanced"])
def test_max_numel_smaller_than_a_segment_truncates_like_the_reference_grid(balanced):
    gs, ls, ln = [0, 2000, 2600], [0, 1500, 1100], [1500, 300, 400]
    host_local, host_out = random_values(1800, torch.float32, 1), random_values(3000, torch.float32, 2)
    for max_numel in (1, 256, 257, 300, 1500):
        want = host_out.clone()
        CO.copy_rank_segments_to_full_kernel(host_local, want, gs, ls, ln, max_numel)
        out = host_out.to(DEV)
        run_device(host_local.to(DEV), out, gs, ls, ln, max_numel, balanced)
        assert_same_bits(out, want)


@pytest.mark.parametrize("balanced", [False, True], ids=["uniform", "balanced"])
def test_segments_that_leave_a_tensor_are_skipped(balanced):
    """The host cannot read device metadata; the kernel refuses what would fault instead."""
    host_local, host_out = random_values(100, torch.float32, 1), random_values(100, torch.float32, 2)
    gs = [0, 90, -4, 50, 60, 70]
    ls = [0, 10, 20, 95, -1, 30]
    ln = [10, 11, 5, 6, 5, -3]  # 2nd leaves the output, 3rd / 5th negative starts, 4th leaves local, 6th negative size
    want = host_out.clone()
    want[0:10] = host_local[0:10]
    out = host_out.to(DEV)
    run_device(host_local.to(DEV), out, gs, ls, ln, 16, balanced)
    assert_same_bits(out, want)


def test_empty_inputs_and_reference_error_cases():
    local, out = torch.zeros(8, device=DEV), torch.ones(8, device=DEV)
    empty = torch.zeros(0, dtype=torch.int64, device=DEV)
    N.copy_rank_segments_to_full(local, out, empty, empty, empty, 0)
    meta = torch.zeros(1, dtype=torch.int64, device=DEV)
    N.copy_rank_segments_to_full(local, out, meta, meta, meta + 4, 0)  # max_numel 0: nothing is launched
    assert out.tolist() == [1.0] * 8
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        N.copy_rank_segments_to_full(local.cpu(), out, meta, meta, meta, 1)
    with pytest.raises(RuntimeError, match="must be int64"):
        N.copy_rank_segments_to_full(local, out, meta.int(), meta, meta, 1)
    with pytest.raises(RuntimeError, match="metadata length mismatch"):
        N.copy_rank_segments_to_full(local, out, meta, torch.zeros(2, dtype=torch.int64, device=DEV), meta, 1)
    with pytest.raises(RuntimeError, match="dtype mismatch"):
        N.copy_rank_segments_to_full(local, out.double(), meta, meta, meta, 1)
    with pytest.raises(RuntimeError, match="must be 1D"):
        N.copy_rank_segments_to_full(local.view(2, 4), out, meta, meta, meta, 1)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        N.copy_rank_segments_to_full(local[::2], out, meta, meta, meta, 1)
    with pytest.raises(RuntimeError, match="max_numel must be non-negative"):
        N.copy_rank_segments_to_full(local, out, meta, meta, meta, -1)
    with pytest.raises(RuntimeError, match="workspace of"):
        N.copy_rank_segments_to_full(local, out, meta, meta, meta + 1, 1, workspace=torch.zeros(8, dtype=torch.uint8, device=DEV))


def test_block_shard_rows_of_a_hidden4096_layer_match_the_segment_program():
    """Rank 3 of the 2 x 2 block layout: 42 500 row segments of 2048 or 5504 elements (plus two vector quarters),
    every launch shape against the compiled segment program and the closed form."""
    w = HIDDEN4096_W4_BLOCK
    plan = w.plan()
    rank = 3
    segments = plan.rank_segments[rank]
    local = torch.empty(plan.shard_sizes[rank], dtype=torch.bfloat16, device=DEV).normal_(0, 0.02, generator=torch.Generator(device=DEV).manual_seed(1))
    want = torch.zeros(plan.total_numel, dtype=torch.bfloat16, device=DEV)
    local_segments_program(segments, local.numel(), plan.total_numel, torch.bfloat16, device=DEV).run((local,), want)
    # closed form for one matrix: the rank's block of Wqkv is the strided slice [R/2:, C/2:]
    spec = w.specs[0]
    rows, cols = spec.shape
    assert torch.equal(want[spec.offset : spec.end].view(rows, cols)[rows // 2 :, cols // 2 :].reshape(-1), local[: rows * cols // 4])
    gs, ls, ln, max_numel = N._segment_metadata_tensors(tuple(segments), device=torch.device(DEV))
    assert N._segment_metadata_tensors(tuple(segments), device=torch.device(DEV))[0] is gs  # cached per layout
    for ws in (None, N.copy_rank_segments_workspace(len(segments), DEV)):
        out = torch.zeros_like(want)
        N.copy_rank_segments_to_full(local, out, gs, ls, ln, max_numel, workspace=ws)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_replays_under_graph_capture():
    """Enqueue-only: both launch shapes captured into one HIP graph, every replay checked against the oracle with
    the program's own eager work between the replays."""
    rng = np.random.default_rng(11)
    gs, ls, ln, local_n, out_n = random_segments(rng, 64, 3000)
    meta = [torch.tensor(v, dtype=torch.int64, device=DEV) for v in (gs, ls, ln)]
    ws = N.copy_rank_segments_workspace(len(gs), DEV)
    local = torch.empty(local_n, dtype=torch.bfloat16, device=DEV)
    out_a, out_b = (torch.empty(out_n, dtype=torch.bfloat16, device=DEV) for _ in range(2))

    def enqueue():
        N.copy_rank_segments_to_full(local, out_a, *meta, max(ln))
        N.copy_rank_segments_to_full(local, out_b, *meta, max(ln), workspace=ws)

    enqueue()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for seed in (10, 20, 30):
        host_local, host_out = random_values(local_n, torch.bfloat16, seed), random_values(out_n, torch.bfloat16, seed + 1)
        local.copy_(host_local)
        out_a.copy_(host_out)
        out_b.copy_(host_out)
        graph.replay()
        torch.cuda.synchronize()
        want = host_out.clone()
        CO.copy_rank_segments_to_full_kernel(host_local, want, gs, ls, ln, max(ln))
        assert_same_bits(out_a, want)
        assert_same_bits(out_b, want)
        (local.float() * 2).sum().item()
