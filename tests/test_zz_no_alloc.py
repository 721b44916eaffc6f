"""The entry point that allocates nothing (``mfsdp_copy_rank_segments_to_full_noalloc``): called through the C ABI
and checked bit for bit against ``mfsdp_copy_rank_segments_to_full_device`` with a caller's workspace, on two calls
in a row that share the library's static scratch, the second with a smaller input."""
import ctypes

import numpy as np
import pytest
import torch

from matrix_fsdp_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def layout(rng, n_seg, max_len):
    lengths = [int(rng.integers(0, max_len + 1)) for _ in range(n_seg)]
    lengths[n_seg // 2] = 40 * max_len + 3  # one long segment beside the short ones
    local_starts, cursor = [], 1
    for n in lengths:
        local_starts.append(cursor)
        cursor += n + int(rng.integers(0, 3))
    global_starts, gcursor = [0] * n_seg, 2
    for i in rng.permutation(n_seg):
        global_starts[i] = gcursor
        gcursor += lengths[i] + int(rng.integers(0, 3))
    return global_starts, local_starts, lengths, cursor, gcursor


def call(name, local, out, meta, n_seg, max_numel, *extra):
    lib = _lib.lib()
    stream = torch.cuda.current_stream(out.device).cuda_stream
    rc = getattr(lib, name)(
        local.data_ptr(), local.numel(), out.data_ptr(), out.numel(), meta[0].data_ptr(), meta[1].data_ptr(), meta[2].data_ptr(),
        n_seg, max_numel, local.element_size(), *extra, stream,
    )
    return rc


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.uint8], ids=lambda d: str(d).split(".")[-1])
def test_two_calls_in_a_row_match_the_workspace_entry_point(dtype):
    rng = np.random.default_rng(21)
    torch.cuda.set_device(DEV)
    free_before = None
    for n_seg, max_len in ((900, 700), (37, 90)):  # the second call is smaller: stale tile counts lie behind its own
        gs, ls, ln, local_n, out_n = layout(rng, n_seg, max_len)
        meta = [torch.tensor(v, dtype=torch.int64, device=DEV) for v in (gs, ls, ln)]
        gen = torch.Generator().manual_seed(n_seg)
        local = torch.randint(0, 251, (local_n,), generator=gen).to(dtype).to(DEV)
        base = torch.randint(0, 251, (out_n,), generator=gen).to(dtype).to(DEV)
        want, have = base.clone(), base.clone()
        ws = torch.empty(int(_lib.lib().mfsdp_copy_rank_segments_workspace_bytes(n_seg)), dtype=torch.uint8, device=DEV)
        _lib.check(call("mfsdp_copy_rank_segments_to_full_device", local, want, meta, n_seg, max(ln), ws.data_ptr(), ws.numel()))
        torch.cuda.synchronize()
        if free_before is None:
            # a first call loads the code object (and with it the static array); from here on nothing may be allocated
            _lib.check(call("mfsdp_copy_rank_segments_to_full_noalloc", local, have.clone(), meta, n_seg, max(ln)))
            torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _lib.check(call("mfsdp_copy_rank_segments_to_full_noalloc", local, have, meta, n_seg, max(ln)))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert not torch.equal(have, base)
        view = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[have.element_size()]
        assert torch.equal(have.view(view), want.view(view))


def test_more_segments_than_the_static_scratch_holds_are_rejected():
    torch.cuda.set_device(DEV)
    n_seg = _lib.NOALLOC_MAX_SEGMENTS + 1
    meta = [torch.zeros(n_seg, dtype=torch.int64, device=DEV) for _ in range(3)]
    local, out = torch.zeros(8, device=DEV), torch.ones(8, device=DEV)
    rc = call("mfsdp_copy_rank_segments_to_full_noalloc", local, out, meta, n_seg, 4)
    assert rc == 3  # MFSDP_ERR_UNSUPPORTED
    assert b"at most 131071 segments" in _lib.lib().mfsdp_last_error()
    with pytest.raises(RuntimeError, match="at most 131071 segments"):
        _lib.check(rc)
    torch.cuda.synchronize()
    assert out.tolist() == [1.0] * 8
    # the largest count it accepts runs (all segments empty: nothing is written)
    meta = [m[: n_seg - 1] for m in meta]
    _lib.check(call("mfsdp_copy_rank_segments_to_full_noalloc", local, out, meta, n_seg - 1, 4))
    torch.cuda.synchronize()
    assert out.tolist() == [1.0] * 8
