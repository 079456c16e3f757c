"""Builds and loads tests/lds_fill.hip (test support, not part of the product)."""

from __future__ import annotations

import ctypes
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "lds_fill.hip")
LIB = os.path.join(HERE, "liblds_fill.so")


def build(force: bool = True) -> str:
    if force or not os.path.exists(LIB):
        hipcc = "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else "hipcc"
        r = subprocess.run(
            [hipcc, "--offload-arch=gfx950", "-O2", "-shared", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-o", LIB, SRC],
            capture_output=True, text=True,
        )  # (the host pass warns that it does not know the target feature: harmless)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {SRC}:\n{r.stderr}")
    return LIB


def load():
    if not os.path.exists(LIB):
        raise RuntimeError(f"{LIB} is missing: run __graft_entry__.build() (or tests.lds_fill.build()) first")
    lib = ctypes.CDLL(LIB)
    lib.lds_fill.restype = ctypes.c_int
    lib.lds_fill.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    return lib
