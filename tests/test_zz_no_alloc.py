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


def test_replays_under_graph_capture_after_a_first_call_outside_it():
    """The callers this entry point is for capture it into a HIP graph.  Its first call on a device looks the static
    array's address up (and loads the code object), which belongs outside a capture; from the second call on it only
    enqueues kernels.  Every replay is checked against the workspace entry point run eagerly, with the program's own
    eager work and synchronisations between the replays."""
    rng = np.random.default_rng(33)
    torch.cuda.set_device(DEV)
    n_seg, max_len = 300, 500
    gs, ls, ln, local_n, out_n = layout(rng, n_seg, max_len)
    meta = [torch.tensor(v, dtype=torch.int64, device=DEV) for v in (gs, ls, ln)]
    ws = torch.empty(int(_lib.lib().mfsdp_copy_rank_segments_workspace_bytes(n_seg)), dtype=torch.uint8, device=DEV)
    local = torch.zeros(local_n, dtype=torch.bfloat16, device=DEV)
    have = torch.zeros(out_n, dtype=torch.bfloat16, device=DEV)
    _lib.check(call("mfsdp_copy_rank_segments_to_full_noalloc", local, have, meta, n_seg, max(ln)))  # outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(call("mfsdp_copy_rank_segments_to_full_noalloc", local, have, meta, n_seg, max(ln)))
    for seed in (1, 2, 3):
        gen = torch.Generator().manual_seed(seed)
        local.copy_(torch.randn(local_n, generator=gen).bfloat16())
        base = torch.randn(out_n, generator=gen).bfloat16().to(DEV)
        have.copy_(base)
        graph.replay()
        torch.cuda.synchronize()
        want = base.clone()
        _lib.check(call("mfsdp_copy_rank_segments_to_full_device", local, want, meta, n_seg, max(ln), ws.data_ptr(), ws.numel()))
        torch.cuda.synchronize()
        assert not torch.equal(have, base)
        assert torch.equal(have.view(torch.int16), want.view(torch.int16))
        (local.float() * 2).sum().item()
