"""Builds the gfx950 shared library ``fairseq2_amd/lib/libfs2moe.so`` with hipcc.

Run as ``python -m fairseq2_amd.build``.  hipcc cross-compiles, so no GPU is
needed to build; the library is loaded with ctypes by :mod:`fairseq2_amd._abi`.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfs2moe.so")

SOURCES = ["abi.hip", "router.hip", "dispatch.hip", "experts.hip", "combine.hip", "backward.hip", "mx.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-f32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
    "-Wno-unknown-warning-option",
]


def hipcc_path() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; the MoE kernels cannot be built")
    return found


def build_library(verbose: bool = True, extra_flags: list[str] | None = None) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, *(extra_flags or [])]
    cmd += ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES]
    cmd += ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
