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
_OUT_HOOKS = os.path.join(_PKG, "libemm_kv_hooks.so")

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
    # the leading scalar kernel arguments arrive in scalar registers when a wave starts (the
    # kernels order their parameters by first use for this): one memory round trip less per wave
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def library_path() -> str:
    return _OUT


def hooks_library_path() -> str:
    return _OUT_HOOKS


def build_library(verbose: bool = False, hooks: bool = False) -> str:
    """Compile csrc/emm_kv.hip (which includes the csrc/*.inc kernel files) -> libemm_kv.so (always recompiles). ``hooks=True`` builds
    libemm_kv_hooks.so instead: the same source with -DEMM_BENCH_HOOKS, which adds the launch-variant
    switch, the memory-system probes and the quotient sweep that bench.py and the GPU tests use
    (csrc/emm_kv_hooks.h, csrc/emm_kv_hooks.inc). The product library never contains them."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = _OUT_HOOKS if hooks else _OUT
    extra = ["-DEMM_BENCH_HOOKS", f"-I{os.path.join(_PKG, 'csrc')}"] if hooks else []
    cmd = [hipcc, *HIPCC_FLAGS, *extra, f"-I{_INC}", "-o", out, _SRC]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}")
    if verbose and proc.stdout:
        print(proc.stdout)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_library(verbose=True, hooks=True))
