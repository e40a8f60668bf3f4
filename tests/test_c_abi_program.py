"""The C ABI used from C: tests/c_abi/c_abi_check.c (no Python, no torch on its path) is compiled with gcc
against include/emm_kv.h, libemm_kv.so and the HIP runtime, and checks every data-moving entry point of the header
(block moves with device and host tables, migrate, the appends of all three layouts in 16-bit and fp8, the
dequantising unpack, concat, the plain copy) against the loops of oracle/kv_oracle.c."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi", "c_abi_check.c")
EXE = os.path.join(ROOT, "tests", "c_abi", "c_abi_check")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build_program() -> str:
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROCM, "include"), "-o", EXE, SRC, os.path.join(ROOT, "oracle", "kv_oracle.c"),
           "-L" + os.path.join(ROOT, "elasticmm_amd"), "-lemm_kv", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../elasticmm_amd", "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    subprocess.check_call(cmd)
    return EXE


def test_c_program_compiles_and_links_against_the_header_and_library():
    assert os.path.exists(os.path.join(ROOT, "elasticmm_amd", "libemm_kv.so")), "libemm_kv.so has not been built"
    build_program()
    assert os.access(EXE, os.X_OK)


@pytest.mark.gpu
def test_c_program_passes_on_the_gpu():
    if not os.path.exists(EXE):
        build_program()
    out = subprocess.run([EXE], capture_output=True, text=True, timeout=110)
    print(out.stdout[-2000:], out.stderr[-2000:], flush=True)
    assert out.returncode == 0 and "C ABI CHECK PASSED" in out.stdout
