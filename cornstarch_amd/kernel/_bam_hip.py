"""ctypes binding of ``libbam_hip.so`` (declarations: ``include/bam_hip.h``).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_DIR, "libbam_hip.so")

BAM_DTYPE_F16 = 0
BAM_DTYPE_BF16 = 1
BAM_MAX_SEQLEN = 4194304
BAM_STATIC_PLAN_BYTES = 8 << 20
ABI_VERSION = 10

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_f32 = ctypes.c_float

class IndexView(ctypes.Structure):
    """``bam_index_view`` of include/bam_hip.h (host struct holding device pointers)."""

    _fields_ = [
        ("q_bits", ctypes.c_void_p),
        ("k_bits", ctypes.c_void_p),
        ("q_pos", ctypes.c_void_p),
        ("k_pos", ctypes.c_void_p),
        ("q_bits_stride_b", ctypes.c_int64),
        ("k_bits_stride_b", ctypes.c_int64),
        ("Sq", ctypes.c_int32),
        ("Sk", ctypes.c_int32),
    ]


class Bias(ctypes.Structure):
    """``bam_bias`` of include/bam_hip.h (host struct holding a device pointer)."""

    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64),
        ("stride_h", ctypes.c_int64),
        ("stride_m", ctypes.c_int64),
        ("is_f32", ctypes.c_int32),
    ]


class Plan(ctypes.Structure):
    """``bam_plan`` of include/bam_hip.h (host struct holding device pointers into the plan workspace)."""

    _fields_ = [
        ("fine", ctypes.c_void_p),
        ("fine_stride_b", ctypes.c_int64),
        ("fine_stride_s", ctypes.c_int64),
        ("order", ctypes.c_void_p),
        ("order_stride_b", ctypes.c_int64),
        ("ds_entry", ctypes.c_void_p),
        ("ds_entry_stride_b", ctypes.c_int64),
        ("ds_tile_base", ctypes.c_void_p),
        ("ds_count", ctypes.c_void_p),
        ("ds_tile_order", ctypes.c_void_p),
        ("group_order", ctypes.c_void_p),
        ("row_workloads", ctypes.c_void_p),
        ("ds_workspace", ctypes.c_void_p),
        ("ds_capacity", ctypes.c_int64),
        ("row_bits", ctypes.c_void_p),
        ("row_bits_stride_b", ctypes.c_int64),
        ("row_bits_stride_n", ctypes.c_int64),
        ("col_bits", ctypes.c_void_p),
        ("col_bits_stride_b", ctypes.c_int64),
        ("col_bits_stride_s", ctypes.c_int64),
        ("B", ctypes.c_int32),
        ("Sq", ctypes.c_int32),
        ("Sk", ctypes.c_int32),
        ("generation", ctypes.c_int32),
    ]


_view = ctypes.POINTER(IndexView)
_bias = ctypes.POINTER(Bias)
_plan = ctypes.POINTER(Plan)

# name -> argtypes, exactly the prototypes of include/bam_hip.h
SIGNATURES = {
    "bam_tile_flags": [_ptr, _i64, _ptr, _i64, _i64, _int, _int, _ptr],
    "bam_materialize_mask": [_ptr, _i64, _ptr, _int, _int, _ptr],
    "bam_tile_plan": [_ptr, _i64, _ptr, _i64, _i64, _ptr, _i64, _int, _int, _plan, _ptr],
    "bam_tile_plan_static": [_ptr, _i64, _ptr, _i64, _i64, _int, _int, _plan, _ptr],
    "bam_fwd": [_ptr] * 7 + [_i64] * 15 + [_int] * 5 + [_f32, _int, _bias, _plan, _ptr],
    "bam_bwd_preprocess": [_ptr] * 3 + [_i64] * 6 + [_int] * 5 + [_ptr],
    "bam_bwd": [_ptr] * 11 + [_i64] * 24 + [_int] * 5 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_bwd_dkdv": [_ptr] * 10 + [_i64] * 21 + [_int] * 5 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_bwd_dq": [_ptr] * 9 + [_i64] * 18 + [_int] * 5 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_mask_tile_flags": [_ptr, _ptr, _i64, _i64, _int, _int, _int, _ptr],
    "bam_mask_tile_plan": [_ptr, _ptr, _i64, _i64, _ptr, _i64, _int, _int, _int, _plan, _ptr],
    "bam_fwd_masked": [_ptr] * 7 + [_i64] * 14 + [_int] * 6 + [_f32, _int, _bias, _plan, _ptr],
    "bam_bwd_dkdv_masked": [_ptr] * 10 + [_i64] * 20 + [_int] * 6 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_bwd_dq_masked": [_ptr] * 9 + [_i64] * 17 + [_int] * 6 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_flag_row_workloads": [_ptr, _i64, _i64, _int, _int, _int, _ptr, _ptr],
    "bam_gather_bitfields": [_ptr, _i64, _int, _ptr, _int, _ptr, _i64, _ptr, _int, _ptr],
    "bam_plan_indexed": [_view, _ptr, _i64, _int, _plan, _ptr],
    "bam_fwd_indexed": [_ptr] * 5 + [_view, _ptr] + [_i64] * 14 + [_int] * 4 + [_f32, _int, _bias, _plan, _ptr],
    "bam_bwd_dkdv_indexed": [_ptr] * 8 + [_view, _ptr] + [_i64] * 20 + [_int] * 4 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_bwd_dq_indexed": [_ptr] * 7 + [_view, _ptr] + [_i64] * 17 + [_int] * 4 + [_f32, _int, _int, _bias, _plan, _ptr],
    "bam_decode": [_ptr] * 4 + [_i64] * 10 + [_int] * 5 + [_f32, _int, _int, _f32, _ptr, _i64, _ptr],
}

_lib = None


class BamError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise BamError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built "
            "(run `python -m cornstarch_amd.build`); there is no fallback path"
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.bam_last_error.restype = ctypes.c_char_p
    lib.bam_last_error.argtypes = []
    lib.bam_abi_version.restype = _int
    lib.bam_abi_version.argtypes = []
    lib.bam_plan_workspace_bytes.restype = _i64
    lib.bam_plan_workspace_bytes.argtypes = [_int, _int]
    lib.bam_plan_workspace_bytes_rect.restype = _i64
    lib.bam_plan_workspace_bytes_rect.argtypes = [_int, _int, _int]
    lib.bam_mask_plan_workspace_bytes.restype = _i64
    lib.bam_mask_plan_workspace_bytes.argtypes = [_int, _int, _int]
    lib.bam_decode_workspace_bytes.restype = _i64
    lib.bam_decode_workspace_bytes.argtypes = [_int] * 6
    lib.bam_ds_workspace_bytes.restype = _i64
    lib.bam_ds_workspace_bytes.argtypes = [_int, _i64]
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _int
    if lib.bam_abi_version() != ABI_VERSION:
        raise BamError(f"libbam_hip.so has ABI {lib.bam_abi_version()}, this binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise BamError(f"{name} failed ({rc}): {lib.bam_last_error().decode()}")
