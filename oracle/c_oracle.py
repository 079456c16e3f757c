"""ctypes loader for the C restatement (``bam_oracle.c``).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "libbam_oracle.so")
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


def build(force: bool = False) -> str:
    """Compile ``bam_oracle.c`` with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _DIR, "libbam_oracle.so"])
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.bam_oracle_allow.argtypes = [_i64, _i64, _i64, _i64]
        L.bam_oracle_allow.restype = ctypes.c_int
        L.bam_oracle_mask.argtypes = [_p, _i64, _i64, _p]
        L.bam_oracle_mask_indexed.argtypes = [_p, _i64, _i64, _p, _i64, _p, _i64, _p]
        L.bam_oracle_tile_flags.argtypes = [_p, _i64, _i64, _p]
        L.bam_oracle_attn_fwd.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, ctypes.c_double, _p, _p]
        L.bam_oracle_delta.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _p]
        L.bam_oracle_attn_bwd.argtypes = [_p] * 7 + [_i64] * 5 + [ctypes.c_double] + [_p] * 3
        for f in ("mask", "mask_indexed", "tile_flags", "attn_fwd", "delta", "attn_bwd"):
            getattr(L, "bam_oracle_" + f).restype = None
        _lib = L
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_p)


def _c(a, dt):
    return np.ascontiguousarray(np.asarray(a), dtype=dt)


def allow(bf_q: int, bf_k: int, i: int, j: int) -> bool:
    return bool(lib().bam_oracle_allow(bf_q, bf_k, i, j))


def mask(bf) -> np.ndarray:
    bf = _c(bf, np.int64)
    B, S = bf.shape
    out = np.empty((B, S, S), dtype=np.uint8)
    lib().bam_oracle_mask(_ptr(bf), B, S, _ptr(out))
    return out.astype(bool)


def mask_indexed(bf, idx_q, idx_k) -> np.ndarray:
    bf, idx_q, idx_k = _c(bf, np.int64), _c(idx_q, np.int64), _c(idx_k, np.int64)
    B, S = bf.shape
    out = np.empty((B, idx_q.size, idx_k.size), dtype=np.uint8)
    lib().bam_oracle_mask_indexed(_ptr(bf), B, S, _ptr(idx_q), idx_q.size, _ptr(idx_k), idx_k.size, _ptr(out))
    return out.astype(bool)


def tile_flags(bf) -> np.ndarray:
    bf = _c(bf, np.int64)
    B, S = bf.shape
    out = np.empty((B, -(-S // 128), -(-S // 32)), dtype=np.int8)
    lib().bam_oracle_tile_flags(_ptr(bf), B, S, _ptr(out))
    return out


def attn_fwd(q, k, v, bf, scale=None):
    q, k, v, bf = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32), _c(bf, np.int64)
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    scale = scale or 1.0 / math.sqrt(D)
    o = np.empty_like(q)
    lse = np.empty((B, Hq, S), dtype=np.float32)
    lib().bam_oracle_attn_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(bf), B, S, Hq, Hkv, D, scale, _ptr(o), _ptr(lse))
    return o, lse


def delta(o, do):
    o, do = _c(o, np.float32), _c(do, np.float32)
    B, S, Hq, D = o.shape
    out = np.empty((B, Hq, S), dtype=np.float32)
    lib().bam_oracle_delta(_ptr(o), _ptr(do), B, S, Hq, D, _ptr(out))
    return out


def attn_bwd(q, k, v, do, lse, dlt, bf, scale=None):
    q, k, v, do = (_c(x, np.float32) for x in (q, k, v, do))
    lse, dlt, bf = _c(lse, np.float32), _c(dlt, np.float32), _c(bf, np.int64)
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    scale = scale or 1.0 / math.sqrt(D)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    lib().bam_oracle_attn_bwd(
        _ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(lse), _ptr(dlt), _ptr(bf), B, S, Hq, Hkv, D, scale,
        _ptr(dq), _ptr(dk), _ptr(dv),
    )
    return dq, dk, dv
