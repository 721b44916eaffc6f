"""Gate in front of the HIP copy kernels, with the reference's signatures.

Mirrors the copy half of matrix_fsdp/kernels/native.py (:47-104, :353-360,
:470-489): ``native_copy_rank_segments_to_full`` and
``native_copy_rank_chunk_from_packed`` return ``True`` when the kernel ran and
``False`` when the caller must run its own slice loop (kernels not enabled by the
environment, tensors not eligible).  The gate keeps the reference's opt-in
variable ``MATRIX_FSDP_ENABLE_NATIVE_COPY_KERNELS`` and kill switch
``MATRIX_FSDP_DISABLE_NATIVE_KERNELS``.  The flat-buffer object of this
package does not go through the gate: it owns its segment programs and has
no slice-loop fallback.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from functools import lru_cache

import torch

from .. import _lib
from ..core.layout import LayoutSegment
from .segment_program import SegmentProgram, local_segments_program

_NATIVE_MODULE_NAME = "matrix_fsdp_amd.libmfsdp_hip"
_DISABLE_NATIVE_ENV = "MATRIX_FSDP_DISABLE_NATIVE_KERNELS"
_ENABLE_NATIVE_COPY_ENV = "MATRIX_FSDP_ENABLE_NATIVE_COPY_KERNELS"
_TRUE = {"1", "true", "yes", "on"}

# (device index, dtype, local numel, output numel, segment triples) -> compiled program; kept for the
# life of the process like the reference's metadata tensors (kernels/native.py:20-23, 470-489).
_SEGMENT_PROGRAM_CACHE: dict[tuple, SegmentProgram] = {}


@dataclass(frozen=True)
class NativeKernelStatus:
    available: bool
    module_name: str = _NATIVE_MODULE_NAME
    reason: str | None = None


@lru_cache(maxsize=1)
def native_kernel_status() -> NativeKernelStatus:
    if os.environ.get(_DISABLE_NATIVE_ENV, "").lower() in _TRUE:
        return NativeKernelStatus(False, reason=f"{_DISABLE_NATIVE_ENV} is set")
    try:
        _lib.lib()
    except Exception as exc:
        return NativeKernelStatus(False, reason=f"{type(exc).__name__}: {exc}")
    return NativeKernelStatus(True)


def native_kernel_available() -> bool:
    return native_kernel_status().available


def native_copy_kernels_enabled() -> bool:
    """Opt-in, as in the reference (kernels/native.py:103-104)."""
    return os.environ.get(_ENABLE_NATIVE_COPY_ENV, "").lower() in _TRUE


def _can_use_native_copy(source: torch.Tensor, destination: torch.Tensor) -> bool:
    return (
        source.is_cuda
        and destination.is_cuda
        and source.is_contiguous()
        and destination.is_contiguous()
        and source.dtype == destination.dtype
    )


def native_copy_rank_segments_to_full(
    local_tensor: torch.Tensor,
    output_tensor: torch.Tensor,
    segments: tuple[LayoutSegment, ...],
) -> bool:
    """``output[g0:g1] = local[l0:l1]`` for this rank's segments, one launch."""
    if not native_copy_kernels_enabled() or not native_kernel_available():
        return False
    if not _can_use_native_copy(local_tensor, output_tensor):
        return False
    if not segments:
        return True
    if local_tensor.dim() != 1 or output_tensor.dim() != 1:
        raise RuntimeError("local_tensor and output_tensor must be 1D")
    key = (
        output_tensor.device.index,
        local_tensor.dtype,
        local_tensor.numel(),
        output_tensor.numel(),
        tuple((s.global_start, s.local_start, s.numel) for s in segments),
    )
    program = _SEGMENT_PROGRAM_CACHE.get(key)
    if program is None:
        program = local_segments_program(
            segments, local_tensor.numel(), output_tensor.numel(), local_tensor.dtype, device=output_tensor.device
        )
        _SEGMENT_PROGRAM_CACHE[key] = program
    program.run((local_tensor,), output_tensor)
    return True


# (device type, device index, segment triples) -> (global_starts, local_starts, numels, max_numel), created once per
# layout and kept for the life of the process, as the reference keeps them (kernels/native.py:20-23, 470-489)
_SEGMENT_METADATA_CACHE: dict[tuple, tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]] = {}


def _segment_metadata_tensors(segments: tuple[LayoutSegment, ...], *, device: torch.device):
    key = (device.type, device.index, tuple((s.global_start, s.local_start, s.numel) for s in segments))
    cached = _SEGMENT_METADATA_CACHE.get(key)
    if cached is None:
        columns = [[s.global_start for s in segments], [s.local_start for s in segments], [s.numel for s in segments]]
        tensors = [torch.tensor(c, dtype=torch.int64, device=device) for c in columns]
        cached = (*tensors, max(columns[2], default=0))
        _SEGMENT_METADATA_CACHE[key] = cached
    return cached


def copy_rank_segments_to_full(
    local_tensor: torch.Tensor,
    output_tensor: torch.Tensor,
    global_starts: torch.Tensor,
    local_starts: torch.Tensor,
    numels: torch.Tensor,
    max_numel: int,
    *,
    workspace: torch.Tensor | None = None,
) -> None:
    """The extension function of the reference, argument for argument
    (kernels/native/matrix_copy.cpp:53-83): device int64 metadata tensors, enqueue
    only on the current stream, the reference's checks as ``RuntimeError``.
    ``workspace`` (uint8, ``mfsdp_copy_rank_segments_workspace_bytes`` long)
    selects the byte-balanced launch shape."""
    for t, name in ((local_tensor, "local_tensor"), (output_tensor, "output_tensor"), (global_starts, "global_starts"),
                    (local_starts, "local_starts"), (numels, "numels")):
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    for t, name in ((global_starts, "global_starts"), (local_starts, "local_starts"), (numels, "numels")):
        if t.dtype != torch.int64:
            raise RuntimeError(f"{name} must be int64")
    if local_tensor.dim() != 1:
        raise RuntimeError("local_tensor must be 1D")
    if output_tensor.dim() != 1:
        raise RuntimeError("output_tensor must be 1D")
    if local_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("source and destination dtype mismatch")
    if global_starts.numel() != local_starts.numel() or global_starts.numel() != numels.numel():
        raise RuntimeError("metadata length mismatch")
    if max_numel < 0:
        raise RuntimeError("max_numel must be non-negative")
    if global_starts.numel() == 0:
        return
    ws_ptr, ws_bytes = (None, 0)
    if workspace is not None:
        if not workspace.is_cuda or not workspace.is_contiguous() or workspace.device != output_tensor.device:
            raise RuntimeError("workspace must be a contiguous CUDA tensor on the output's device")
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    stream = torch.cuda.current_stream(output_tensor.device).cuda_stream
    with torch.cuda.device(output_tensor.device):
        _lib.check(
            _lib.lib().mfsdp_copy_rank_segments_to_full_device(
                local_tensor.data_ptr(), local_tensor.numel(), output_tensor.data_ptr(), output_tensor.numel(),
                global_starts.data_ptr(), local_starts.data_ptr(), numels.data_ptr(), global_starts.numel(), int(max_numel),
                local_tensor.element_size(), ws_ptr, ws_bytes, stream,
            )
        )


def copy_rank_segments_workspace(n_segments: int, device) -> torch.Tensor:
    """Scratch for the byte-balanced launch shape of ``copy_rank_segments_to_full``."""
    return torch.empty(int(_lib.lib().mfsdp_copy_rank_segments_workspace_bytes(n_segments)), dtype=torch.uint8, device=device)


def native_copy_rank_chunk_from_packed(
    packed_rank_chunks: torch.Tensor,
    output_tensor: torch.Tensor,
    shard_sizes: tuple[int, ...],
    rank: int,
    *,
    compact: bool,
) -> bool:
    """``output = packed[offset : offset + output.numel()]`` with ``offset`` the
    compact or padded start of rank ``rank``'s chunk."""
    if not native_copy_kernels_enabled() or not native_kernel_available():
        return False
    if not _can_use_native_copy(packed_rank_chunks, output_tensor):
        return False
    if packed_rank_chunks.dim() != 1 or output_tensor.dim() != 1:
        raise RuntimeError("input_tensor and output_tensor must be 1D")
    offset = sum(shard_sizes[:rank]) if compact else rank * max(shard_sizes)
    copy_range(packed_rank_chunks, output_tensor, offset)
    return True


def copy_range(input_tensor: torch.Tensor, output_tensor: torch.Tensor, input_offset: int) -> None:
    """``mfsdp_copy_range`` on the current stream; raises ``RuntimeError`` on
    the reference's error cases (kernels/native/matrix_copy.cpp:85-99)."""
    if not (input_tensor.is_cuda and output_tensor.is_cuda):
        raise RuntimeError("input_tensor and output_tensor must be CUDA tensors")
    if not (input_tensor.is_contiguous() and output_tensor.is_contiguous()):
        raise RuntimeError("input_tensor and output_tensor must be contiguous")
    if input_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("source and destination dtype mismatch")
    stream = torch.cuda.current_stream(output_tensor.device).cuda_stream
    with torch.cuda.device(output_tensor.device):
        _lib.check(
            _lib.lib().mfsdp_copy_range(
                input_tensor.data_ptr(),
                input_tensor.numel(),
                output_tensor.data_ptr(),
                output_tensor.numel(),
                int(input_offset),
                input_tensor.element_size(),
                stream,
            )
        )


_ACCUMULATE_DTYPES = {torch.float32: _lib.DT_F32, torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16}


def accumulate(destination: torch.Tensor, source: torch.Tensor) -> torch.Tensor:
    """``destination += source`` (``mfsdp_accumulate``) on the current stream:
    float32, bfloat16 or float16, both contiguous, same dtype and size."""
    if not (destination.is_cuda and source.is_cuda) or destination.device != source.device:
        raise RuntimeError("destination and source must be CUDA tensors on one device")
    if not (destination.is_contiguous() and source.is_contiguous()):
        raise RuntimeError("destination and source must be contiguous")
    if destination.dtype != source.dtype or destination.dtype not in _ACCUMULATE_DTYPES:
        raise RuntimeError(f"accumulate adds float32, bfloat16 or float16 tensors of one dtype, got {destination.dtype} += {source.dtype}")
    if destination.numel() != source.numel():
        raise RuntimeError(f"destination has {destination.numel()} elements, source has {source.numel()}")
    stream = torch.cuda.current_stream(destination.device).cuda_stream
    with torch.cuda.device(destination.device):
        _lib.check(
            _lib.lib().mfsdp_accumulate(destination.data_ptr(), source.data_ptr(), destination.numel(), _ACCUMULATE_DTYPES[destination.dtype], stream)
        )
    return destination


_CAST_CODES = {
    (torch.bfloat16, torch.float32): _lib.CONVERT_BF16_TO_F32,
    (torch.float32, torch.bfloat16): _lib.CONVERT_F32_TO_BF16,
    (torch.float16, torch.float32): _lib.CONVERT_F16_TO_F32,
    (torch.float32, torch.float16): _lib.CONVERT_F32_TO_F16,
}


def cast(source: torch.Tensor, dtype: torch.dtype, out: torch.Tensor | None = None) -> torch.Tensor:
    """``source.to(dtype)`` for bfloat16 / float16 <-> float32 on the HIP cast kernel;
    returns ``source`` itself when nothing changes, as the reference's
    ``_maybe_to_*_dtype`` helpers do (runtime/flat_buffer.py:1186-1206)."""
    if source.dtype == dtype or not source.is_floating_point():
        return source
    code = _CAST_CODES.get((source.dtype, dtype))
    if code is None:
        raise RuntimeError(f"HIP cast supports bfloat16 / float16 <-> float32, got {source.dtype} -> {dtype}")
    if not source.is_cuda or not source.is_contiguous():
        raise RuntimeError("cast source must be a contiguous CUDA tensor")
    if out is None:
        out = torch.empty(source.shape, dtype=dtype, device=source.device)
    elif out.dtype != dtype or out.numel() != source.numel() or not out.is_contiguous() or out.device != source.device:
        raise RuntimeError("cast output must be contiguous, on the source's device, of the target dtype and size")
    stream = torch.cuda.current_stream(source.device).cuda_stream
    with torch.cuda.device(source.device):
        _lib.check(_lib.lib().mfsdp_cast(source.data_ptr(), out.data_ptr(), source.numel(), code, stream))
    return out
