"""In-tree build of libemm_kv.so with hipcc for gfx950.

The shared object is written next to this file so that it travels with the
source tree; nothing is installed and no JIT cache is used.
"""
from __future__ import annotations

import os
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
_SRC = os.path.join(_PKG, "csrc", "emm_kv.hip")
_INC = os.path.join(_ROOT, "include")
_OUT = os.path.join(_PKG, "libemm_kv.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # bit-exact arithmetic: no fused multiply-add / fused multiply-convert (the fp8 rule is
    # "round the fp32 product, then round to 16 bits", two roundings)
    "-ffp-contract=off",
    # keep the compiler from forming packed-fp32 ops out of float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def library_path() -> str:
    return _OUT


def build_library(verbose: bool = False) -> str:
    """Compile csrc/emm_kv.hip -> libemm_kv.so (always recompiles)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, *HIPCC_FLAGS, f"-I{_INC}", "-o", _OUT, _SRC]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}")
    if verbose and proc.stdout:
        print(proc.stdout)
    return _OUT


if __name__ == "__main__":
    print(build_library(verbose=True))
