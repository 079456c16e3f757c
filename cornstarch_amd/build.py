"""Builds ``libbam_hip.so`` (the HIP kernels + C ABI) for gfx950 with hipcc.

The library has no dependency on torch or Python: plain ``hipcc -shared``.  It is built
in-tree, next to this file, so that the very same binary is what tests, the smoke check
and the benchmark load.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libbam_hip.so")
# the longest compilations first: they are spread over the workers
SOURCES = ["bwd_long.hip", "bwd_dkdv.hip", "bwd_dkdv_save.hip", "bwd_dq_saved.hip", "bwd_dq.hip", "fwd_long.hip", "fwd.hip", "tile_flags.hip", "decode.hip", "bam_abi.hip"]
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # no NaN is ever produced on purpose (masked scores are -inf, never NaN), so max/min need no
    # NaN-quieting canonicalisation instructions
    "-fno-honor-nans",
    # packed fp32 VALU ops are kept off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: libbam_hip.so cannot be built")


def build_library(force: bool = True, verbose: bool = False) -> str:
    """Compile every kernel file and link the shared library.  Returns its path."""
    if not force and os.path.exists(LIB_PATH):
        return LIB_PATH
    hipcc = _hipcc()
    objdir = os.path.join(PKG_DIR, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
        if verbose:
            sys.stderr.write(r.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, verbose="-v" in sys.argv))
