"""CPU oracle for the flat-buffer copy-in / copy-out path.  TEST INFRASTRUCTURE.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product never routes through it.

Each function restates, as plain per-segment slice copies on CPU tensors,
one function of the reference (cited per function).  Plans are duck-typed:
anything with ``total_numel``, ``shard_sizes`` and ``rank_segments`` whose
segments have ``global_start`` / ``global_end`` / ``local_start``.

Pinning (what makes this oracle trustworthy, see tests/test_oracle_*.py):
  * every function is checked against the literal vectors of the reference's
    own tests, committed as tests/golden/reference_vectors.json;
  * chunk-cat is checked against the library routine ``torch._chunk_cat``;
  * the 2x2 block layout is checked against the strided-slice closed form;
  * casts are checked against ``Tensor.to`` over crafted bit patterns;
  * round trips and write-exactly-once invariants on random layouts;
  * ``copy_rank_segments_to_full_kernel`` is checked against a literal thread
    by thread walk of the reference kernel's grid on small inputs, and against
    ``copy_local_rank_segments`` (pinned by the reference vectors) whenever
    ``max_numel`` covers every segment;
  * the checkpoint redistribution (``target_local_shard_from_full`` etc.) is
    checked against the pinned pack / unpack functions: a rank's shard of the
    full buffer is that rank's slice of the packed order, on random layouts.
"""
from __future__ import annotations

import torch


def _numel(seg) -> int:
    return seg.global_end - seg.global_start


def rank_packed_offset(shard_sizes, rank: int) -> int:
    """matrix_fsdp/runtime/flat_buffer.py:1362-1363."""
    return sum(shard_sizes[:rank])


# ---------------------------------------------------------------- P1
def pack_full_tensor_by_rank_segments(full: torch.Tensor, plan) -> torch.Tensor:
    """full flat buffer -> compact rank-major shards
    (matrix_fsdp/runtime/flat_buffer.py:1304-1316)."""
    full = full.reshape(-1)
    if full.numel() != plan.total_numel:
        raise RuntimeError(f"Full tensor has {full.numel()} elements, expected {plan.total_numel}.")
    packed = full.new_empty(sum(plan.shard_sizes))
    for rank, segments in enumerate(plan.rank_segments):
        base = rank_packed_offset(plan.shard_sizes, rank)
        for seg in segments:
            dst = base + seg.local_start
            packed[dst : dst + _numel(seg)].copy_(full[seg.global_start : seg.global_end])
    return packed


# ---------------------------------------------------------------- P2
def pad_rank_shard(local: torch.Tensor, max_shard: int) -> torch.Tensor:
    """Zero-padded all-gather staging of one rank's shard
    (matrix_fsdp/runtime/collectives.py:236-237, 248-249)."""
    padded = local.new_zeros(max_shard)
    padded[: local.numel()].copy_(local)
    return padded


def gather_padded(rank_shards: list[torch.Tensor], shard_sizes) -> torch.Tensor:
    """What ``all_gather_into_tensor`` of every rank's padded shard leaves in
    the gathered buffer: slot ``r`` = rank r's shard, tail zero
    (matrix_fsdp/runtime/collectives.py:236-241)."""
    max_shard = max(shard_sizes, default=0)
    return torch.cat([pad_rank_shard(s, max_shard) for s in rank_shards]) if rank_shards else torch.empty(0)


# ---------------------------------------------------------------- P3
def unpad_gathered(gathered_padded: torch.Tensor, shard_sizes, out: torch.Tensor | None = None) -> torch.Tensor:
    """padded gathered ``[W*max]`` -> compact ``[sum shard_sizes]``
    (matrix_fsdp/runtime/collectives.py:264-272)."""
    max_shard = max(shard_sizes, default=0)
    if out is None:
        out = gathered_padded.new_empty(sum(shard_sizes))
    offset = 0
    for rank, size in enumerate(shard_sizes):
        out[offset : offset + size].copy_(gathered_padded[rank * max_shard : rank * max_shard + size])
        offset += size
    return out


# ---------------------------------------------------------------- P4
def packed_rank_shards_are_full_tensor_order(plan) -> bool:
    """matrix_fsdp/runtime/flat_buffer.py:1335-1353."""
    if plan.total_numel != sum(plan.shard_sizes):
        return False
    if plan.rank_segments is None:
        return True
    for rank, segments in enumerate(plan.rank_segments):
        base = rank_packed_offset(plan.shard_sizes, rank)
        cursor = 0
        for seg in segments:
            if seg.local_start != cursor:
                return False
            if seg.global_start != base + seg.local_start or seg.global_end != base + seg.local_start + _numel(seg):
                return False
            cursor = seg.local_start + _numel(seg)
        if cursor != plan.shard_sizes[rank]:
            return False
    return True


def unpack_rank_shards_to_full_tensor(rank_shards: torch.Tensor, plan) -> torch.Tensor:
    """compact rank-major shards -> full flat buffer; the *same tensor* comes
    back when rank-major order already is full order
    (matrix_fsdp/runtime/flat_buffer.py:1318-1333)."""
    rank_shards = rank_shards.reshape(-1)
    expected = sum(plan.shard_sizes)
    if rank_shards.numel() != expected:
        raise RuntimeError(f"Packed rank shards have {rank_shards.numel()} elements, expected {expected}.")
    if packed_rank_shards_are_full_tensor_order(plan):
        return rank_shards
    full = rank_shards.new_empty(plan.total_numel)
    for rank, segments in enumerate(plan.rank_segments):
        base = rank_packed_offset(plan.shard_sizes, rank)
        for seg in segments:
            src = base + seg.local_start
            full[seg.global_start : seg.global_end].copy_(rank_shards[src : src + _numel(seg)])
    return full


# ---------------------------------------------------------------- P6
def copy_local_rank_segments(local: torch.Tensor, output: torch.Tensor, segments) -> None:
    """One rank's shard -> its slots of the full buffer
    (matrix_fsdp/runtime/collectives.py:495-503;
    matrix_fsdp/kernels/native/matrix_copy_cuda.cu:8-23)."""
    for seg in segments:
        output[seg.global_start : seg.global_end].copy_(local[seg.local_start : seg.local_start + _numel(seg)])


def copy_rank_segments_to_full_kernel(local: torch.Tensor, output: torch.Tensor, global_starts, local_starts, numels, max_numel: int) -> None:
    """The extension function as its kernel executes it
    (matrix_fsdp/kernels/native/matrix_copy_cuda.cu:8-23, 38-51): a grid of
    ``ceil(max_numel / 256)`` blocks of 256 threads per segment, thread
    ``offset`` copying one element when ``offset < numel``.  With
    ``max_numel >= max(numels)`` (what the caller passes,
    kernels/native.py:484) this is ``copy_local_rank_segments``; a smaller
    ``max_numel`` leaves the tail of longer segments uncopied."""
    covered = (int(max_numel) + 255) // 256 * 256
    for g, l, n in zip(global_starts, local_starts, numels):
        n = min(int(n), covered)
        if n > 0:
            output[int(g) : int(g) + n].copy_(local[int(l) : int(l) + n])


# ---------------------------------------------------------------- P7
def copy_rank_chunk_from_packed(packed: torch.Tensor, output: torch.Tensor, shard_sizes, rank: int, *, compact: bool) -> None:
    """``output = packed[offset : offset + shard_sizes[rank]]`` with the offset
    rule of matrix_fsdp/kernels/native.py:92
    (kernel: matrix_fsdp/kernels/native/matrix_copy_cuda.cu:25-36)."""
    offset = sum(shard_sizes[:rank]) if compact else rank * max(shard_sizes)
    output.copy_(packed[offset : offset + output.numel()])


# ---------------------------------------------------------------- G4
def maybe_cast(tensor: torch.Tensor, dtype: torch.dtype | None) -> torch.Tensor:
    """``Tensor.to(dtype)`` only for floating tensors whose dtype differs
    (matrix_fsdp/runtime/flat_buffer.py:1186-1206)."""
    if dtype is None or tensor.dtype == dtype or not tensor.is_floating_point():
        return tensor
    return tensor.to(dtype=dtype)


# ---------------------------------------------------------------- G1-G3
def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def classify_copy_in_layout(params, grads, shard_sizes, rank_segments, total_numel) -> str:
    """``flat_contiguous`` / ``fsdp2_chunk`` / ``generic_segment``
    (matrix_fsdp/runtime/grad_bucket.py:119-187).  ``params`` have
    ``offset`` / ``end`` / ``numel``; ``grads`` are the matching tensors."""
    world = len(shard_sizes)

    def flat_ok() -> bool:
        if not params or len(set(shard_sizes)) != 1:
            return False
        cursor = 0
        for size, segments in zip(shard_sizes, rank_segments):
            if len(segments) != 1:
                return False
            seg = segments[0]
            if seg.local_start != 0 or seg.global_start != cursor or seg.global_end != cursor + size:
                return False
            cursor = seg.global_end
        if cursor != total_numel:
            return False
        cursor = 0
        for p, g in zip(params, grads):
            if p.offset != cursor or p.end != cursor + p.numel or g.numel() != p.numel:
                return False
            cursor = p.end
        return cursor == total_numel

    def chunk_ok() -> bool:
        if not params or world == 0:
            return False
        cursor, table = 0, []
        for p, g in zip(params, grads):
            if g.numel() != p.numel or p.end != p.offset + p.numel:
                return False
            size = _ceil_div(p.numel, world)
            table.append((p, cursor, size))
            cursor += size
        if max(shard_sizes, default=0) != cursor or any(s != cursor for s in shard_sizes):
            return False
        for rank in range(world):
            expected = []
            for p, local_start, size in table:
                start = p.offset + rank * size
                end = min(p.end, start + size)
                if start < end:
                    expected.append((start, end, local_start))
            have = [(s.global_start, s.global_end, s.local_start) for s in rank_segments[rank]]
            if have != expected:
                return False
        return True

    if flat_ok():
        return "flat_contiguous"
    if chunk_ok():
        return "fsdp2_chunk"
    return "generic_segment"


def chunk_cat(grads: list[torch.Tensor], world: int, out_2d: torch.Tensor) -> None:
    """Semantics of ``torch._chunk_cat(grads, 0, W, out=out_2d)`` as the
    reference calls it (matrix_fsdp/runtime/grad_bucket.py:200-202): each
    1-D grad of ``n`` elements is cut in ``W`` chunks of ``ceil(n/W)``; row
    ``r`` of the output is the concatenation of every grad's chunk ``r``,
    short or missing chunks zero-padded; the output dtype converts."""
    col = 0
    for g in grads:
        g = g.reshape(-1)
        size = _ceil_div(g.numel(), world)
        for r in range(world):
            piece = g[r * size : min(g.numel(), (r + 1) * size)]
            out_2d[r, col : col + piece.numel()].copy_(piece)
            out_2d[r, col + piece.numel() : col + size].zero_()
        col += size
    if col != out_2d.shape[1]:
        raise RuntimeError("chunk_cat output width does not match the grads.")


def copy_param_grad_to_rank_chunks(packed_2d: torch.Tensor, param, grad: torch.Tensor, rank_segments) -> None:
    """matrix_fsdp/runtime/grad_bucket.py:209-225."""
    for rank, segments in enumerate(rank_segments):
        for seg in segments:
            start = max(param.offset, seg.global_start)
            end = min(param.end, seg.global_end)
            if start >= end:
                continue
            dst = seg.local_start + start - seg.global_start
            packed_2d[rank, dst : dst + (end - start)].copy_(grad[start - param.offset : end - param.offset])


def fill_reduce_scatter_input(
    params, grads, shard_sizes, rank_segments, total_numel, packed: torch.Tensor, *, backend: str = "auto"
) -> torch.Tensor:
    """Dispatcher of matrix_fsdp/runtime/grad_bucket.py:71-116, with the
    reduce-dtype cast of matrix_fsdp/runtime/flat_buffer.py:612 applied to
    each grad first (``packed.dtype`` is the reduce dtype)."""
    world = len(shard_sizes)
    if world == 0:
        raise ValueError("MatrixGradBucket requires at least one rank.")
    max_shard = max(shard_sizes, default=0)
    if packed.ndim != 1:
        raise ValueError(f"packed must be 1D, got shape {tuple(packed.shape)}.")
    if packed.numel() != world * max_shard:
        raise ValueError(f"packed has {packed.numel()} elements, expected {world * max_shard}.")
    if backend not in ("auto", "flat_cat", "foreach_copy", "chunk_cat", "segment_copy"):
        raise ValueError("backend must be 'auto', 'flat_cat', 'foreach_copy', 'chunk_cat', or 'segment_copy'.")
    grads = [maybe_cast(g.reshape(-1), packed.dtype) for g in grads]
    kind = classify_copy_in_layout(params, grads, shard_sizes, rank_segments, total_numel)
    if backend in ("flat_cat", "foreach_copy") and kind != "flat_contiguous":
        raise ValueError(f"{backend} backend requires an equal, rank-contiguous flat bucket layout.")
    if backend == "chunk_cat" and kind != "fsdp2_chunk":
        raise ValueError("chunk_cat backend requires an FSDP2-style per-parameter chunk bucket layout.")
    if backend == "foreach_copy":
        for p, g in zip(params, grads):
            packed[p.offset : p.end].copy_(g)
        return packed
    if backend == "flat_cat" or (backend == "auto" and kind == "flat_contiguous"):
        torch.cat(grads, out=packed)
        return packed
    if backend == "chunk_cat" or (backend == "auto" and kind == "fsdp2_chunk"):
        chunk_cat(grads, world, packed.view(world, max_shard))
        return packed
    packed.zero_()
    packed_2d = packed.view(world, max_shard)
    for p, g in zip(params, grads):
        if g.numel() != p.numel:
            raise RuntimeError(f"Gradient for {p.fqn} has {g.numel()} elements, expected {p.numel}.")
        copy_param_grad_to_rank_chunks(packed_2d, p, g, rank_segments)
    return packed


# ---------------------------------------------------------------- G5
def packed_grad_offset_for_param(param, shard_sizes, rank_segments, *, compact: bool) -> int | None:
    """Where a whole parameter's grad sits in the rank-chunk workspace, or
    ``None`` when it is not one contiguous run there
    (matrix_fsdp/runtime/flat_buffer.py:1274-1302)."""
    max_shard = max(shard_sizes, default=0)
    cursor = 0
    start: int | None = None
    end: int | None = None
    for rank, segments in enumerate(rank_segments):
        for seg in segments:
            g0 = max(param.offset, seg.global_start)
            g1 = min(param.end, seg.global_end)
            if g0 >= g1:
                continue
            if g0 - param.offset != cursor:
                return None
            base = rank_packed_offset(shard_sizes, rank) if compact else rank * max_shard
            cur = base + seg.local_start + g0 - seg.global_start
            if start is None:
                start = cur
            elif end != cur:
                return None
            end = cur + (g1 - g0)
            cursor = g1 - param.offset
    if start is None or cursor != param.numel:
        return None
    return start


def fill_compact_owner_reduce_scatter_input(params, grads, shard_sizes, rank_segments, packed: torch.Tensor) -> torch.Tensor:
    """Whole-parameter owner layouts: zero the compact ``[sum shard_sizes]``
    workspace and drop every grad at ``rank_base(owner) + local_start``
    (matrix_fsdp/runtime/flat_buffer.py:1232-1252)."""
    expected = sum(shard_sizes)
    if packed.ndim != 1:
        raise ValueError(f"packed_rank_chunks must be 1D, got shape {tuple(packed.shape)}.")
    if packed.numel() != expected:
        raise ValueError(f"packed_rank_chunks has {packed.numel()} elements, expected {expected}.")
    packed.zero_()
    for p, g in zip(params, grads):
        g = maybe_cast(g.reshape(-1), packed.dtype)
        if g.numel() != p.numel:
            raise RuntimeError(f"Gradient for {p.fqn} has {g.numel()} elements, expected {p.numel}.")
        off = packed_grad_offset_for_param(p, shard_sizes, rank_segments, compact=True)
        if off is None:
            raise RuntimeError(f"Gradient for {p.fqn} cannot be packed into compact owner rank chunks.")
        packed[off : off + p.numel].copy_(g)
    return packed


# ---------------------------------------------------------------- fused forms the GPU path is compared with
def pack_to_padded(full: torch.Tensor, plan) -> torch.Tensor:
    """P1 then P2 for every simulated rank: the gathered, padded buffer
    ``[W*max_shard]`` the all-gather would deliver."""
    packed = pack_full_tensor_by_rank_segments(full, plan)
    shards, off = [], 0
    for size in plan.shard_sizes:
        shards.append(packed[off : off + size])
        off += size
    return gather_padded(shards, plan.shard_sizes)


def unpack_from_padded(gathered_padded: torch.Tensor, plan) -> torch.Tensor:
    """P3 then P4: padded gathered buffer -> full flat buffer."""
    return unpack_rank_shards_to_full_tensor(unpad_gathered(gathered_padded, plan.shard_sizes), plan)


def param_views(full: torch.Tensor, params) -> list[torch.Tensor]:
    """P5: ``full[offset:end].view(shape)`` per parameter, aliasing ``full``
    (matrix_fsdp/runtime/flat_buffer.py:413-425)."""
    return [full[p.offset : p.end].view(p.shape) for p in params]


# ---------------------------------------------------------------- checkpoint load into another layout
def target_local_shard_from_full(full: torch.Tensor, local_segments) -> torch.Tensor:
    """One rank's shard of a full flat tensor: its segments' slices, concatenated
    in segment order (matrix_fsdp/checkpoint/state_dict.py:1330-1345)."""
    if not local_segments:
        return full.new_empty(0)
    return torch.cat([full[seg.global_start : seg.global_end] for seg in local_segments])


def target_local_param_tensor_from_full(full_param: torch.Tensor, param_segments, param_offset: int) -> torch.Tensor:
    """One rank's part of a parameter-shaped tensor (an optimizer moment) given
    flat over the whole parameter; ``param_segments`` are the rank's segments
    of that parameter in flat-buffer coordinates
    (matrix_fsdp/checkpoint/state_dict.py:1348-1363)."""
    if not param_segments:
        return full_param.new_empty(0)
    return torch.cat([full_param[seg.global_start - param_offset : seg.global_end - param_offset] for seg in param_segments])


def full_from_source_rank_shards(source_shards: list[torch.Tensor]) -> torch.Tensor:
    """The reference's reassembly of a saved flat buffer: the source ranks'
    shards concatenated in rank order (state_dict.py:934-939).  Equal to the
    full buffer only when the saved layout is rank-ordered; otherwise the
    packed order has to be unpacked along the saved segments
    (``unpack_rank_shards_to_full_tensor``)."""
    return torch.cat([shard.reshape(-1) for shard in source_shards])
