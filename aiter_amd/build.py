"""Builds ``libaiter_fp8bs.so`` (the C-ABI library) in-tree with hipcc for gfx950.

Usage: ``python -m aiter_amd.build`` (always recompiles), or ``build_library()`` from Python.
The library has no torch / Python dependency; it links only against the HIP runtime.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libaiter_fp8bs.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

SOURCES = ["abi.hip", "workspace.hip", "norm_quant_kernels.hip", "gemm_blockscale_kernels.hip", "gemm_prefill.hip", "gemm_decode.hip",
           "gemm_mid.hip", "moe_kernels.hip"]

# -ffp-contract=off: the quantiser's rounding sequence must stay one IEEE operation per step.
# The packed-fp32 target feature is switched off for device code on purpose; the host pass
# does not know the feature and says so, which is harmless.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH)")


def _compile(src: str, obj_dir: str, verbose: bool) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return obj


def build_library(verbose: bool = False) -> str:
    """Compile every HIP translation unit and link the shared library. Returns its path."""
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir, verbose), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
