"""ctypes binding of libmfsdp_hip.so (the C ABI declared in include/mfsdp_hip.h).

The library is looked up beside this package only.  There is no CPU fallback:
when it is missing, ``lib()`` raises and every operator built on it fails.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libmfsdp_hip.so")

OK = 0
CONVERT_NONE = 0
CONVERT_BF16_TO_F32 = 1
CONVERT_F32_TO_BF16 = 2
CONVERT_F16_TO_F32 = 3
CONVERT_F32_TO_F16 = 4
DT_F32 = 0
DT_BF16 = 1
DT_F16 = 2  # mfsdp_accumulate only
ABI_VERSION = 6
MUON_SHARED_MACHINE = 1
NOALLOC_MAX_SEGMENTS = 131071  # MFSDP_NOALLOC_MAX_SEGMENTS


class CopyRun(Structure):
    """``mfsdp_copy_run``."""

    _fields_ = [
        ("src_off", c_int64),
        ("dst_off", c_int64),
        ("row_len", c_int64),
        ("rows", c_int64),
        ("src_stride", c_int64),
        ("dst_stride", c_int64),
        ("src_id", c_int32),
        ("reserved", c_int32),
    ]


# name -> (restype, argtypes); every symbol include/mfsdp_hip.h declares
SIGNATURES = {
    "mfsdp_last_error": (c_char_p, []),
    "mfsdp_abi_version": (c_int, []),
    "mfsdp_copy_range": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "mfsdp_copy_rank_segments_to_full": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), c_int64, c_int, c_void_p],
    ),
    "mfsdp_copy_rank_segments_workspace_bytes": (c_int64, [c_int64]),
    "mfsdp_copy_rank_segments_to_full_device": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p],
    ),
    "mfsdp_copy_rank_segments_to_full_noalloc": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p],
    ),
    "mfsdp_merge_segment_runs": (c_int64, [POINTER(CopyRun), c_int64, POINTER(CopyRun)]),
    "mfsdp_segment_program_create": (
        c_int,
        [POINTER(CopyRun), c_int64, POINTER(c_int64), c_int32, c_int64, c_int, c_int, POINTER(c_void_p)],
    ),
    "mfsdp_segment_program_destroy": (None, [c_void_p]),
    "mfsdp_segment_program_bytes": (c_int64, [c_void_p]),
    "mfsdp_segment_program_num_runs": (c_int64, [c_void_p]),
    "mfsdp_segment_program_run": (c_int, [c_void_p, POINTER(c_void_p), c_int32, c_void_p, c_void_p]),
    "mfsdp_segment_program_run_many": (c_int, [c_void_p, c_int32, POINTER(c_void_p), c_int32, POINTER(c_void_p), c_void_p]),
    "mfsdp_set_copy_tuning": (None, [c_int, c_int, c_int, c_int]),
    "mfsdp_hbm_probe": (c_int, [c_int, c_void_p, c_void_p, c_int64, c_void_p]),
    "mfsdp_cast": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "mfsdp_muon_workspace_bytes": (c_int64, [c_int64, c_int64]),
    "mfsdp_muon_executed_flops": (c_int64, [c_int64, c_int64, c_int, c_int]),
    "mfsdp_newton_schulz": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_float, c_float, c_float, c_int, c_float, c_void_p, c_void_p, c_int64, c_void_p],
    ),
    "mfsdp_muon_step": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_double, c_double, c_double, c_int,
         c_float, c_float, c_float, c_int, c_float, c_double, c_void_p, c_int64, c_void_p],
    ),
    "mfsdp_muon_step_ex": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_double, c_double, c_double, c_int,
         c_float, c_float, c_float, c_int, c_float, c_double, c_int, c_void_p, c_int64, c_void_p],
    ),
    "mfsdp_set_muon_tuning": (None, [c_int, c_int, c_int, c_int, c_int]),
    "mfsdp_gemm_nt_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "mfsdp_accumulate": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "mfsdp_adamw_step": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_double, c_double, c_double, c_double, c_double, c_void_p],
    ),
    "mfsdp_adamw_step_ex": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_double, c_double, c_double, c_double, c_double, c_int, c_void_p],
    ),
}

_LIB = None


class NativeLibraryError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Loads the library once; raises ``NativeLibraryError`` when it is absent
    or its ABI version differs from this binding's."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `python matrix-fsdp_amd/csrc/build.py` "
            "(there is no CPU fallback for the HIP path)."
        )
    handle = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)  # AttributeError here means the library is stale
        fn.restype = restype
        fn.argtypes = argtypes
    if handle.mfsdp_abi_version() != ABI_VERSION:
        raise NativeLibraryError(
            f"{LIB_PATH} has ABI version {handle.mfsdp_abi_version()}, this binding expects {ABI_VERSION}: rebuild it."
        )
    _LIB = handle
    return handle


def check(status: int) -> None:
    """Non-zero status -> ``RuntimeError`` with the library's message (the
    reference's TORCH_CHECK convention, matrix_fsdp/kernels/native/matrix_copy.cpp:60-78)."""
    if status != OK:
        message = lib().mfsdp_last_error()
        raise RuntimeError(f"libmfsdp_hip: {message.decode() if message else 'error'} (code {status})")
