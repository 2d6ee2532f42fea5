"""The C ABI called from a program written in plain C (no Python, no torch in the process).

`avelang_amd/abi_check` is built by the package's Makefile from `csrc/host_check/abi_check.c`: it includes only
`include/ave_fp4.h` and the HIP runtime API, runs a 96 x 160 x 512 MXFP4 GEMM with unit scales on every kernel
variant and compares each bf16 result with the integer-exact value it computes on the host.  This is what a
compiled-language binding of the library goes through; it stands beside this package's Python caller
(`avelang_amd/amdgpu_gemm_fp4.py`), which mirrors the reference's host wrapper
(reference python/avelang_kernels/amdgpu_gemm.py:458-494).
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "..", "avelang_amd", "abi_check")


@pytest.mark.gpu
def test_plain_c_caller_gets_exact_results():
    assert os.path.exists(BINARY), "avelang_amd/abi_check is missing: run `make -C avelang_amd/csrc`"
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "abi_check: ok" in done.stdout
