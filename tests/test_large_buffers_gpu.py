"""Buffers past 2^31: element offsets that do not fit 32 bits, and runs of more than 2^31 vector groups (which the
host splits into several device runs).  Expected values come from torch slicing on the same device; the sizes are
far beyond what the CPU oracle copies in reasonable time, and the layouts are the ones it is pinned on."""
import numpy as np
import pytest
import torch

from matrix_fsdp_amd.core.plans import block_grid_plan, fsdp2_chunk_plan
from matrix_fsdp_amd.kernels.segment_program import RUN_DTYPE, SegmentProgram, pack_program, unpack_program
from matrix_fsdp_amd.workloads import param_specs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def random_bits(numel: int, dtype: torch.dtype, seed: int) -> torch.Tensor:
    """``numel`` elements of ``dtype`` with random bit patterns, filled in 1 GiB pieces."""
    gen = torch.Generator(device=DEV).manual_seed(seed)
    out = torch.empty(numel, dtype=dtype, device=DEV)
    raw = out.view(torch.uint8)
    step = 1 << 30
    for start in range(0, raw.numel(), step):
        raw[start : start + step].random_(0, 256, generator=gen)
    return out


@pytest.fixture(autouse=True)
def free_cached_blocks():
    torch.cuda.empty_cache()
    yield
    torch.cuda.empty_cache()


def test_element_offsets_past_two_to_the_31():
    """A 32768 x 65536 bf16 matrix (2^31 elements) followed by a vector: every offset of the vector is past 2^31."""
    specs = param_specs([("embed.weight", (32768, 65536)), ("norm.weight", (1 << 22,))])
    total = specs[-1].end
    assert total > 2**31
    full = random_bits(total, torch.bfloat16, 1).view(torch.int16)  # compared as bit patterns
    for plan in (fsdp2_chunk_plan(specs, 4), block_grid_plan(specs, (2, 2))):
        padded = torch.empty(4 * plan.max_shard_size, dtype=torch.int16, device=DEV)
        pack_program(plan, torch.int16, device=DEV).run((full,), padded)
        matrix = full[: specs[0].numel].view(32768, 65536)
        vector = full[specs[0].numel :]
        for r in range(4):
            slot = padded[r * plan.max_shard_size : (r + 1) * plan.max_shard_size]
            if len(plan.rank_segments[r]) == 2:  # row chunks
                want_matrix = matrix[r * 8192 : (r + 1) * 8192].reshape(-1)
            else:  # block (i, j)
                i, j = divmod(r, 2)
                want_matrix = matrix[i * 16384 : (i + 1) * 16384, j * 32768 : (j + 1) * 32768].reshape(-1)
            assert torch.equal(slot[: want_matrix.numel()], want_matrix)
            assert torch.equal(slot[want_matrix.numel() :], vector[r * (1 << 20) : (r + 1) * (1 << 20)])
            del want_matrix
        out = torch.zeros(total, dtype=torch.int16, device=DEV)
        unpack_program(plan, torch.int16, device=DEV).run((padded,), out)
        assert torch.equal(out, full)
        del padded, out


def test_runs_of_more_than_two_to_the_31_groups_are_split():
    """Odd byte offsets force 1-byte vector groups, so a run of 2^31 + 12345 bytes holds more groups than one
    device run may (the row lookup divides by multiply-high, exact below 2^31) and is cut along its length; three
    rows of 2^30 bytes each exceed the limit together and are cut by rows."""
    long_len = 2**31 + 12345
    src = random_bits(long_len + 64, torch.uint8, 2)
    runs = np.zeros(1, dtype=RUN_DTYPE)
    runs["src_off"], runs["dst_off"], runs["row_len"], runs["rows"], runs["src_id"] = 1, 3, long_len, 1, 0
    dst = torch.full((long_len + 8,), 7, dtype=torch.uint8, device=DEV)
    SegmentProgram(runs, [src.numel()], dst.numel(), src_dtype=torch.uint8, device=DEV).run((src,), dst)
    assert torch.equal(dst[3 : 3 + long_len], src[1 : 1 + long_len])
    assert dst[:3].tolist() == [7, 7, 7] and dst[3 + long_len :].tolist() == [7] * 5
    del dst

    row, rows, src_stride, dst_stride = 2**30, 3, 2**30 + 3, 2**30 + 5
    src = random_bits(rows * src_stride + 8, torch.uint8, 3)
    runs = np.zeros(1, dtype=RUN_DTYPE)
    runs["src_off"], runs["dst_off"], runs["row_len"], runs["rows"], runs["src_id"] = 1, 1, row, rows, 0
    runs["src_stride"], runs["dst_stride"] = src_stride, dst_stride
    dst = torch.full((rows * dst_stride + 8,), 9, dtype=torch.uint8, device=DEV)
    SegmentProgram(runs, [src.numel()], dst.numel(), src_dtype=torch.uint8, device=DEV, merge=False).run((src,), dst)
    for r in range(rows):
        assert torch.equal(dst[1 + r * dst_stride : 1 + r * dst_stride + row], src[1 + r * src_stride : 1 + r * src_stride + row])
        assert dst[1 + r * dst_stride + row : 1 + r * dst_stride + row + 4].tolist() == [9] * 4  # the gap between rows is untouched
